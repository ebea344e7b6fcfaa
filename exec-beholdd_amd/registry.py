"""One registry from an architecture's name (config.json `architectures[0]`) to its model.

The reference dispatches on the checkpoint's architecture tag by exact match and names the
implemented set when the tag is unknown (crates/beholdd-model/src/qwen3moe.rs:476-495).
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Callable

from .config.base import ConfigError, architecture_name


@dataclass(frozen=True)
class ArchitectureEntry:
    name: str
    config_class: type
    build: Callable       # build(config) -> model (no weights yet)


_ARCHITECTURES: dict = {}


def register_architecture(name: str, config_class: type, build: Callable) -> ArchitectureEntry:
    if name in _ARCHITECTURES:
        raise ValueError(f"architecture {name!r} is already registered")
    entry = ArchitectureEntry(name, config_class, build)
    _ARCHITECTURES[name] = entry
    return entry


def unregister_architecture(name: str) -> None:
    _ARCHITECTURES.pop(name, None)


def registered_architectures() -> list[str]:
    return sorted(_ARCHITECTURES)


def resolve_architecture(config_dict: dict, origin: str = "config.json") -> ArchitectureEntry:
    name = architecture_name(config_dict, origin)
    entry = _ARCHITECTURES.get(name)
    if entry is None:
        raise ConfigError(f"{origin}: unsupported architecture {name!r}; implemented architectures are "
                          + ", ".join(registered_architectures()))
    return entry


def configuration_of(entry: ArchitectureEntry, config_dict: dict, origin: str = "config.json", model_dir=None):
    """The architecture's typed configuration of a config.json.  A configuration class that says `needs_shapes` takes sizes
    that only a tensor's shape gives from the checkpoint's header (name -> shape, no payload is read) as `shapes`; without a
    model folder it gets None and has to find those sizes in the dictionary itself."""
    if not getattr(entry.config_class, "needs_shapes", False):
        return entry.config_class.from_dict(config_dict, origin)
    shapes = None
    if model_dir is not None:
        import os

        from .weights.safetensors_io import SafetensorsReader
        if os.path.isdir(model_dir) and any(name.endswith(".safetensors") for name in os.listdir(model_dir)):
            reader = SafetensorsReader(model_dir)
            try:
                shapes = {name: tuple(item.shape) for name, item in reader.entries.items()}
            finally:
                reader.close()
    return entry.config_class.from_dict(config_dict, origin, shapes=shapes)
