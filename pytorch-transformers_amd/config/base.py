"""Base class of typed model configurations read from ``config.json``.

The reference turns the JSON dict into keyword arguments of the config class
and keeps keys it does not know as plain attributes
(src/transformers/configuration_utils.py:213-324, from_dict :714-772).  Here a
configuration is a dataclass: known keys become typed fields, unknown keys are
kept in ``extra`` and written back on save, and ``validate()`` rejects
combinations that the reference would only fail on later.
"""
from __future__ import annotations

import dataclasses
import json
import os
from typing import Any, ClassVar, Dict

CONFIG_NAME = "config.json"  # src/transformers/utils/__init__.py:254


class ConfigError(ValueError):
    """A configuration that cannot be built into a model."""


@dataclasses.dataclass
class ModelConfig:
    """Fields every architecture shares (src/transformers/configuration_utils.py:213-324)."""

    model_type: ClassVar[str] = ""
    #: legacy key -> field name, applied before the fields are filled
    key_aliases: ClassVar[Dict[str, str]] = {}

    tie_word_embeddings: bool = True  # configuration_utils.py:223-225
    torch_dtype: Any = None
    architectures: Any = None
    pad_token_id: Any = None
    bos_token_id: Any = None
    eos_token_id: Any = None
    use_cache: bool = True
    extra: Dict[str, Any] = dataclasses.field(default_factory=dict)

    def __post_init__(self):
        self.normalize()
        self.validate()

    # hooks -------------------------------------------------------------
    def normalize(self) -> None:
        """Fill fields whose default depends on other fields."""

    def validate(self) -> None:
        """Raise ConfigError for values no model can be built from."""

    # dict / json -------------------------------------------------------
    @classmethod
    def preprocess_dict(cls, d: Dict[str, Any]) -> Dict[str, Any]:
        """Rewrite legacy keys; subclasses extend."""
        out = dict(d)
        for old, new in cls.key_aliases.items():
            if old in out:
                val = out.pop(old)
                out[new] = val
        return out

    @classmethod
    def from_dict(cls, d: Dict[str, Any], **overrides) -> "ModelConfig":
        d = cls.preprocess_dict({**d, **overrides})
        mt = d.pop("model_type", cls.model_type)
        if mt != cls.model_type:
            raise ConfigError(f"config.json says model_type={mt!r}, but {cls.__name__} is for {cls.model_type!r}")
        names = {f.name for f in dataclasses.fields(cls) if f.name != "extra"}
        known = {k: v for k, v in d.items() if k in names}
        extra = {k: v for k, v in d.items() if k not in names}
        return cls(**known, extra=extra)

    @classmethod
    def from_json_file(cls, path: str, **overrides) -> "ModelConfig":
        with open(path, "r", encoding="utf-8") as f:
            return cls.from_dict(json.load(f), **overrides)

    @classmethod
    def from_pretrained(cls, folder: str, **overrides) -> "ModelConfig":
        return cls.from_json_file(os.path.join(folder, CONFIG_NAME), **overrides)

    def to_dict(self) -> Dict[str, Any]:
        d = {"model_type": self.model_type}
        for f in dataclasses.fields(self):
            if f.name == "extra":
                continue
            d[f.name] = getattr(self, f.name)
        d.update(self.extra)
        if d.get("torch_dtype") is not None:
            d["torch_dtype"] = str(d["torch_dtype"]).replace("torch.", "")
        return d

    def to_json_string(self) -> str:
        return json.dumps(self.to_dict(), indent=2, sort_keys=True) + "\n"

    def save_pretrained(self, folder: str) -> None:
        os.makedirs(folder, exist_ok=True)
        with open(os.path.join(folder, CONFIG_NAME), "w", encoding="utf-8") as f:
            f.write(self.to_json_string())
