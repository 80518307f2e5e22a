"""Typed model configurations and the registry from an architecture's name to its model.

A configuration class reads the keys of its own architecture's ``config.json``; nothing
that the file gives is repeated as a constant in code.  ``register_architecture`` binds
the name that ``config.json`` carries in ``architectures[0]`` to a configuration class
and a function that builds the model from it, which is the role of kappai's static
``k_registry`` (src/arch.c:12-139) and its ``RECIPE_REGISTER`` (src/recipe.h:577-580).
"""
from __future__ import annotations

import json
from dataclasses import dataclass, fields
from pathlib import Path
from typing import Any, Callable, Dict, List, Optional, Union


class ConfigError(ValueError):
    """A config.json that cannot describe a model of its architecture."""


_MISSING = object()


class KeyReader:
    """Reads typed keys from a config.json dictionary and reports what is missing, as
    kappai's ``req_i32``/``req_f32`` getters do for GGUF keys (src/model.c:98-111)."""

    def __init__(self, raw: Dict[str, Any], where: str = "config.json"):
        self.raw = raw
        self.where = where

    def _get(self, key, default):
        """``key``: a name, or several names for the same thing of which the first present one
        counts (checkpoints of one architecture written by different versions of its tools)."""
        names = (key,) if isinstance(key, str) else tuple(key)
        for name in names:
            if name in self.raw and self.raw[name] is not None:
                return self.raw[name]
        if default is _MISSING:
            also = "" if len(names) == 1 else " (also read as " + ", ".join(
                f"'{n}'" for n in names[1:]) + ")"
            raise ConfigError(f"{self.where}: required key '{names[0]}' is missing{also}")
        return default

    @staticmethod
    def _name(key) -> str:
        return key if isinstance(key, str) else key[0]

    def int(self, key, default=_MISSING) -> Optional[int]:
        v = self._get(key, default)
        if v is None:
            return None
        if isinstance(v, bool) or not isinstance(v, (int, float)) or int(v) != v:
            raise ConfigError(f"{self.where}: key '{self._name(key)}' must be an integer, got {v!r}")
        return int(v)

    def int_or_ints(self, key, default=_MISSING):
        """One integer or a list of them (checkpoints write ``eos_token_id`` either way)."""
        v = self._get(key, default)
        if v is None:
            return None
        items = v if isinstance(v, (list, tuple)) else [v]
        for x in items:
            if isinstance(x, bool) or not isinstance(x, (int, float)) or int(x) != x:
                raise ConfigError(f"{self.where}: key '{self._name(key)}' must be an integer or a "
                                  f"list of integers, got {v!r}")
        return [int(x) for x in items] if isinstance(v, (list, tuple)) else int(v)

    def float(self, key, default=_MISSING) -> Optional[float]:
        v = self._get(key, default)
        if v is None:
            return None
        if isinstance(v, bool) or not isinstance(v, (int, float)):
            raise ConfigError(f"{self.where}: key '{self._name(key)}' must be a number, got {v!r}")
        return float(v)

    def bool(self, key, default=_MISSING) -> bool:
        v = self._get(key, default)
        if not isinstance(v, bool):
            raise ConfigError(f"{self.where}: key '{self._name(key)}' must be true or false, got {v!r}")
        return v

    def list(self, key, default=_MISSING):
        v = self._get(key, default)
        if v is None:
            return None
        if not isinstance(v, (list, tuple)):
            raise ConfigError(f"{self.where}: key '{self._name(key)}' must be a list, got {v!r}")
        return list(v)


@dataclass
class ModelConfig:
    """What every architecture's configuration offers to the rest of the engine."""

    architecture: str
    # What the engine reads beside ``vocab_size``.  An architecture whose config.json gives them
    # fills them in from its own keys; the defaults mean "the file says nothing".
    max_position_embeddings: int = 0                       # longest sequence; 0: none named
    eos_token_id: Optional[Union[int, List[int]]] = None   # token(s) that end a generation

    # -- to be provided by the architecture -------------------------------------------
    @classmethod
    def from_dict(cls, raw: Dict[str, Any]) -> "ModelConfig":
        raise NotImplementedError

    def to_dict(self) -> Dict[str, Any]:
        """The config.json keys this configuration was read from."""
        raise NotImplementedError

    @property
    def vocab_size(self) -> int:  # pragma: no cover - overridden by dataclass fields
        raise NotImplementedError

    def describe(self) -> str:
        return ", ".join(f"{f.name}={getattr(self, f.name)!r}" for f in fields(self))


@dataclass
class Architecture:
    name: str
    config_cls: type
    build_model: Callable[..., Any]


_ARCHITECTURES: Dict[str, Architecture] = {}


def register_architecture(name: str, config_cls: type, build_model: Callable[..., Any]) -> None:
    """Bind ``architectures[0]`` of a config.json to a configuration class and a model
    builder ``build_model(config, dtype) -> Model``."""
    _ARCHITECTURES[name] = Architecture(name, config_cls, build_model)


def _load_builtin_architectures() -> None:
    """The package's own architectures register themselves when ``kappai_amd.models`` is
    imported; make sure that has happened before a name is looked up."""
    from .. import models  # noqa: F401


def known_architectures():
    _load_builtin_architectures()
    return sorted(_ARCHITECTURES)


def lookup_architecture(name: str) -> Architecture:
    """Unknown names are an error that lists what is known (kappai: "unrecognized
    architecture", src/arch.c:126-139)."""
    _load_builtin_architectures()
    if name not in _ARCHITECTURES:
        raise ConfigError(
            f"unrecognized architecture '{name}'; known: {', '.join(known_architectures()) or 'none'}")
    return _ARCHITECTURES[name]


def architecture_name(raw: Dict[str, Any]) -> str:
    archs = raw.get("architectures")
    if not isinstance(archs, list) or not archs or not isinstance(archs[0], str):
        raise ConfigError("config.json: key 'architectures' must be a list that starts with the "
                          "model class name")
    return archs[0]


def config_from_dict(raw: Dict[str, Any]) -> ModelConfig:
    arch = lookup_architecture(architecture_name(raw))
    return arch.config_cls.from_dict(raw)


def load_config(model_dir) -> ModelConfig:
    path = Path(model_dir) / "config.json"
    if not path.is_file():
        raise ConfigError(f"{path}: no config.json in the model folder")
    try:
        raw = json.loads(path.read_text())
    except json.JSONDecodeError as exc:
        raise ConfigError(f"{path}: not valid JSON ({exc})") from exc
    if not isinstance(raw, dict):
        raise ConfigError(f"{path}: top level must be an object")
    return config_from_dict(raw)
