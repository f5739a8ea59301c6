"""One registry from an architecture's name (``config.json``'s ``architectures[0]``, or its ``architecture``) to
its typed configuration.  A configuration expands into a model specification, and every
architecture is run by the same :class:`~torchlet_amd.models.decoder.DecoderModel`, so
adding an architecture means adding a configuration class (and parts, if it needs new ones).
"""
from __future__ import annotations

import json
from pathlib import Path

from .config.base import ConfigError, ModelConfig
from .config.bafulorn import BafulornConfig
from .config.fotovik import FotovikConfig
from .config.migurax import MiguraxConfig
from .config.nebutar import NebutarConfig
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
register_architecture(MiguraxConfig)
register_architecture(NebutarConfig)
register_architecture(FotovikConfig)
register_architecture(BafulornConfig)


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
    return config_class(architecture_of(d, str(path))).from_dict(d)


def architecture_of(d: dict, where: str = "config.json") -> str:
    """The architecture a ``config.json`` names: the first entry of its list ``architectures``, or its string ``architecture``."""
    archs = d.get("architectures")
    if isinstance(archs, list) and archs:
        return archs[0]
    if isinstance(d.get("architecture"), str) and d["architecture"]:
        return d["architecture"]
    raise ConfigError(f"{where}: 'architectures' must be a non-empty list (or 'architecture' a name)")
