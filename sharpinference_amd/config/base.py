"""Typed model configuration: the base class and the reader of ``config.json``.

A configuration class owns every size and constant that a model folder's
``config.json`` gives; code elsewhere takes them from the configuration object and
holds none of its own.  The class for a folder is found through the architecture
registry by ``architectures[0]``, as the reference picks its hyper-parameter set
from ``general.architecture`` (reference: src/SharpInference.Core/ModelGraph.cs:259-265).
"""
from __future__ import annotations

import json
import os
from dataclasses import dataclass, fields
from typing import Any, Dict, Optional, Tuple


class ConfigError(ValueError):
    """A config.json that cannot describe a model: the message names the key."""


def special_tokens_from(src: Dict[str, Any]) -> Dict[str, Any]:
    """eos_token_id (absent, one id or a list of ids) and bos_token_id of a config.json, as the
    keyword arguments of a configuration class."""
    eos = src.get("eos_token_id")
    try:
        ids = () if eos is None else tuple(int(t) for t in eos) if isinstance(eos, (list, tuple)) else (int(eos),)
        bos = None if src.get("bos_token_id") is None else int(src["bos_token_id"])
    except (TypeError, ValueError):
        raise ConfigError(f"eos_token_id / bos_token_id must be token ids (got {eos!r}, {src.get('bos_token_id')!r})") from None
    return {"eos_token_ids": ids, "bos_token_id": bos}


@dataclass
class ModelConfig:
    """Base of all architecture configurations."""

    architecture: str = ""
    # what ends a generation (config.json's eos_token_id: one id or a list) and what starts a prompt
    eos_token_ids: Tuple[int, ...] = ()
    bos_token_id: Optional[int] = None

    # -- reading ---------------------------------------------------------
    @classmethod
    def from_dict(cls, d: Dict[str, Any]) -> "ModelConfig":  # pragma: no cover - abstract
        raise NotImplementedError

    def to_dict(self) -> Dict[str, Any]:  # pragma: no cover - abstract
        raise NotImplementedError

    def validate(self) -> None:
        """Raise ConfigError when sizes or options contradict each other."""

    def special_tokens_dict(self) -> Dict[str, Any]:
        """The token keys as config.json writes them (absent where the configuration has none)."""
        out: Dict[str, Any] = {}
        if self.eos_token_ids:
            out["eos_token_id"] = list(self.eos_token_ids) if len(self.eos_token_ids) > 1 else self.eos_token_ids[0]
        if self.bos_token_id is not None:
            out["bos_token_id"] = self.bos_token_id
        return out

    # -- helpers ---------------------------------------------------------
    def replace(self, **changes) -> "ModelConfig":
        values = {f.name: getattr(self, f.name) for f in fields(self)}
        values.update(changes)
        out = type(self)(**values)
        out.validate()
        return out


def read_config_dict(model_dir_or_file: str) -> Dict[str, Any]:
    path = model_dir_or_file
    if os.path.isdir(path):
        path = os.path.join(path, "config.json")
    if not os.path.isfile(path):
        raise ConfigError(f"no config.json at {path}")
    with open(path, "r", encoding="utf-8") as f:
        try:
            d = json.load(f)
        except json.JSONDecodeError as e:
            raise ConfigError(f"{path}: not valid JSON ({e})") from None
    if not isinstance(d, dict):
        raise ConfigError(f"{path}: top level must be an object")
    return d


def architecture_name(d: Dict[str, Any]) -> str:
    archs = d.get("architectures")
    if isinstance(archs, (list, tuple)) and archs and isinstance(archs[0], str):
        return archs[0]
    raise ConfigError("config.json has no 'architectures' list naming the model class")


def load_config(source) -> ModelConfig:
    """config.json (a folder, a file or a dict already read) -> typed configuration."""
    from ..registry import get_architecture

    d = source if isinstance(source, dict) else read_config_dict(source)
    arch = get_architecture(architecture_name(d))
    cfg = arch.config_cls.from_dict(d)
    cfg.validate()
    return cfg


def save_config(cfg: ModelConfig, model_dir: str) -> str:
    os.makedirs(model_dir, exist_ok=True)
    path = os.path.join(model_dir, "config.json")
    with open(path, "w", encoding="utf-8") as f:
        json.dump(cfg.to_dict(), f, indent=2)
        f.write("\n")
    return path
