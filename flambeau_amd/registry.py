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
    """``(Architecture, typed config)`` of a model folder.  A configuration class with ``sizes_from_tensors(raw, shapes)``
    is given the shapes of the folder's tensors first (read from the files' headers), for sizes that no key of
    config.json holds."""
    raw = read_config_json(model_dir)
    where = f"{model_dir}/config.json"
    arch = find_architecture(architecture_name(raw, where))
    fill = getattr(arch.config_class, "sizes_from_tensors", None)
    if fill is not None:
        from .weights.loader import SafetensorsDir, WeightFileError
        try:
            src = SafetensorsDir(model_dir)
        except WeightFileError:
            src = None                  # (a folder without weights: the configuration must then say everything itself)
        if src is not None:
            try:
                raw = fill(raw, {name: tuple(src.info(name)[0]) for name in src.names()})
            finally:
                src.close()
    return arch, arch.config_class.from_dict(raw, where)


def _load_builtin():
    from . import models
    models.discover()           # every module under models/ registers its architecture
