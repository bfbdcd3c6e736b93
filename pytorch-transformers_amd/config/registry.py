"""One registry: architecture name -> configuration class and model builder.

The reference keeps two lazy tables keyed by ``model_type``
(src/transformers/models/auto/configuration_auto.py:112, :763-815 and
src/transformers/models/auto/modeling_auto.py:506) and lets users add to them
(``AutoConfig.register`` configuration_auto.py:1102-1116,
``_BaseAutoModelClass.register`` auto_factory.py:573-589).  Here it is one
table.  A *builder* is a function ``builder(config) -> ModelSpec`` (see
``engine.spec``): it lists the blocks, the order they run in, what the cache
holds for them and the tensors the weight file must have.
"""
from __future__ import annotations

import json
import os
from typing import Callable, Dict, Sequence, Tuple, Type

from .base import CONFIG_NAME, ConfigError, ModelConfig

_REGISTRY: Dict[str, Tuple[Type[ModelConfig], Callable]] = {}
_ALIASES: Dict[str, str] = {}  # other names a config.json may give an architecture -> its registered name


def register(model_type: str, config_cls: Type[ModelConfig], builder: Callable, *, exist_ok: bool = False,
             aliases: Sequence[str] = ()) -> None:
    """Add an architecture.  ``aliases`` are further values of ``model_type`` that older files of the same
    architecture carry; they are read as ``model_type``."""
    if not exist_ok and model_type in _REGISTRY:
        raise ValueError(f"model_type {model_type!r} is already registered")
    for a in aliases:
        if not exist_ok and (a in _REGISTRY or _ALIASES.get(a, model_type) != model_type):
            raise ValueError(f"alias {a!r} of {model_type!r} is already taken")
    if getattr(config_cls, "model_type", None) != model_type:
        raise ValueError(
            f"{config_cls.__name__}.model_type is {getattr(config_cls, 'model_type', None)!r}, "
            f"it must equal the registered name {model_type!r}")  # configuration_auto.py:1110-1115
    _REGISTRY[model_type] = (config_cls, builder)
    for a in aliases:
        _ALIASES[a] = model_type


def unregister(model_type: str) -> None:
    _REGISTRY.pop(model_type, None)
    for a in [a for a, t in _ALIASES.items() if t == model_type]:
        del _ALIASES[a]


def resolve_alias(model_type: str) -> str:
    return _ALIASES.get(model_type, model_type)


def known_model_types():
    return sorted(_REGISTRY)


def lookup(model_type: str) -> Tuple[Type[ModelConfig], Callable]:
    try:
        return _REGISTRY[model_type]
    except KeyError:
        # configuration_auto.py:1073-1087
        raise ConfigError(
            f"model_type {model_type!r} is not registered; known types: {', '.join(known_model_types()) or '(none)'}"
        ) from None


class AutoConfig:
    """``AutoConfig.from_pretrained(folder)``: the typed configuration that config.json names."""

    register = staticmethod(register)

    @staticmethod
    def for_model(model_type: str, **kwargs) -> ModelConfig:
        return lookup(model_type)[0](**kwargs)

    @staticmethod
    def from_dict(d: dict, **overrides) -> ModelConfig:
        d = dict(d)
        if "model_type" not in d:
            raise ConfigError("config.json has no 'model_type' key; cannot choose an architecture")
        d["model_type"] = resolve_alias(d["model_type"])
        cls, _ = lookup(d["model_type"])
        return cls.from_dict(d, **overrides)

    @staticmethod
    def from_pretrained(folder: str, **overrides) -> ModelConfig:
        path = os.path.join(folder, CONFIG_NAME)
        if not os.path.isfile(path):
            raise FileNotFoundError(f"no {CONFIG_NAME} in {folder!r}")
        with open(path, "r", encoding="utf-8") as f:
            return AutoConfig.from_dict(json.load(f), **overrides)
