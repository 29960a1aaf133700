"""One registry from an architecture's name (``config.json``'s ``architectures[0]``) to
its typed configuration.  A configuration expands into a model specification, and every
architecture is run by the same :class:`~torchlet_amd.models.decoder.DecoderModel`, so
adding an architecture means adding a configuration class (and parts, if it needs new ones).
"""
from __future__ import annotations

import json
from pathlib import Path

from .config.base import ConfigError, ModelConfig
from .config.qwen2 import Qwen2Config

ARCHITECTURES: dict[str, type[ModelConfig]] = {}


def register_architecture(config_cls: type[ModelConfig]) -> type[ModelConfig]:
    if not config_cls.architecture:
        raise ValueError(f"{config_cls.__name__} names no architecture")
    ARCHITECTURES[config_cls.architecture] = config_cls
    return config_cls


def unregister_architecture(name: str) -> None:
    ARCHITECTURES.pop(name, None)


register_architecture(Qwen2Config)


def config_class(name: str) -> type[ModelConfig]:
    cls = ARCHITECTURES.get(name)
    if cls is None:
        raise ConfigError(f"architecture {name!r} is not registered; known: {', '.join(sorted(ARCHITECTURES))}")
    return cls


def load_config(folder: str | Path) -> ModelConfig:
    """Read ``folder/config.json`` and build the configuration its architecture names."""
    path = Path(folder) / "config.json"
    if not path.exists():
        raise FileNotFoundError(f"no config.json in {folder}")
    d = json.loads(path.read_text())
    archs = d.get("architectures")
    if not isinstance(archs, list) or not archs:
        raise ConfigError(f"{path}: 'architectures' must be a non-empty list")
    return config_class(archs[0]).from_dict(d)
