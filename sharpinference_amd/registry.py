"""The one table from an architecture's name to its configuration class and model builder.

``config.json`` names the model class in ``architectures[0]``; everything that opens a
model folder (the engine, the command line, trace replay) comes through here, as the
reference dispatches on ``general.architecture``
(reference: src/SharpInference.Core/ModelGraph.cs:262, 292-328).
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Callable, Dict

from .config.base import ConfigError


@dataclass
class Architecture:
    name: str
    config_cls: type
    builder: Callable  # builder(config) -> parts.model.DecoderModel (no weights yet)


_ARCHITECTURES: Dict[str, Architecture] = {}


def register_architecture(name: str, config_cls: type, builder: Callable, *, replace: bool = False) -> None:
    if name in _ARCHITECTURES and not replace:
        raise ValueError(f"architecture {name!r} is already registered")
    _ARCHITECTURES[name] = Architecture(name, config_cls, builder)


def unregister_architecture(name: str) -> None:
    _ARCHITECTURES.pop(name, None)


def registered_architectures():
    _ensure_builtin()
    return sorted(_ARCHITECTURES)


def get_architecture(name: str) -> Architecture:
    _ensure_builtin()
    try:
        return _ARCHITECTURES[name]
    except KeyError:
        raise ConfigError(
            f"architecture {name!r} is not registered (known: {', '.join(sorted(_ARCHITECTURES)) or 'none'})"
        ) from None


def build_model(config):
    """Configuration -> a model assembled from parts, still without weights."""
    return get_architecture(config.architecture).builder(config)


_builtin_done = False


def _ensure_builtin() -> None:
    global _builtin_done
    if _builtin_done:
        return
    _builtin_done = True
    from .models import llama4  # noqa: F401  (registers itself)
