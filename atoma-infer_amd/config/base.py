"""Typed reading of ``config.json``.

A model configuration is a frozen dataclass whose fields carry, in their
metadata, the JSON key they are read from, whether the key is required and the
default that applies when it is absent.  ``parse_fields`` turns a JSON object
into the keyword arguments of such a dataclass and reports every problem of the
object in one ``ConfigError``.
"""
from __future__ import annotations

import dataclasses
import json
import os
from typing import Any, Callable, Dict, Optional

_MISSING = dataclasses.MISSING


class ConfigError(ValueError):
    """A config.json that cannot be used; the message lists every fault found."""


def key(name: Optional[str] = None, *, default: Any = _MISSING, convert: Optional[Callable[[Any], Any]] = None,
        doc: str = ""):
    """Declare a dataclass field read from JSON key ``name`` (the field's own name if None).

    A field without ``default`` is required.  ``convert`` receives the raw JSON
    value and returns the typed one, raising ``ValueError``/``TypeError`` on a
    bad value.
    """
    meta = {"json_key": name, "convert": convert, "doc": doc, "required": default is _MISSING}
    if default is _MISSING:
        return dataclasses.field(metadata=meta)
    return dataclasses.field(default=default, metadata=meta)


def as_int(v: Any) -> int:
    if isinstance(v, bool) or not isinstance(v, int):
        raise TypeError(f"expected an integer, got {v!r}")
    return v


def as_positive_int(v: Any) -> int:
    v = as_int(v)
    if v <= 0:
        raise ValueError(f"expected a positive integer, got {v}")
    return v


def as_float(v: Any) -> float:
    if isinstance(v, bool) or not isinstance(v, (int, float)):
        raise TypeError(f"expected a number, got {v!r}")
    return float(v)


def as_bool(v: Any) -> bool:
    if not isinstance(v, bool):
        raise TypeError(f"expected true or false, got {v!r}")
    return v


def optional(conv: Callable[[Any], Any]) -> Callable[[Any], Any]:
    def f(v):
        return None if v is None else conv(v)
    return f


def parse_fields(cls, obj: Dict[str, Any], where: str) -> Dict[str, Any]:
    """Keyword arguments for dataclass ``cls`` from JSON object ``obj``.

    Keys of ``obj`` that ``cls`` does not declare are ignored, as the
    reference's serde structs ignore them (models/src/llama.rs:36-52).
    """
    if not isinstance(obj, dict):
        raise ConfigError(f"{where}: expected a JSON object, got {type(obj).__name__}")
    problems = []
    kwargs: Dict[str, Any] = {}
    for f in dataclasses.fields(cls):
        if "json_key" not in f.metadata:
            continue
        k = f.metadata["json_key"] or f.name
        if k not in obj or (obj[k] is None and not f.metadata["required"]):
            if f.metadata["required"]:
                problems.append(f"missing key '{k}'")
            continue
        conv = f.metadata["convert"]
        try:
            kwargs[f.name] = conv(obj[k]) if conv else obj[k]
        except ConfigError as e:
            problems.append(str(e))
        except (TypeError, ValueError) as e:
            problems.append(f"key '{k}': {e}")
    if problems:
        raise ConfigError(f"{where}: " + "; ".join(problems))
    return kwargs


def read_json(path: str) -> Dict[str, Any]:
    if not os.path.isfile(path):
        raise ConfigError(f"no such file: {path}")
    with open(path, "r", encoding="utf-8") as f:
        try:
            obj = json.load(f)
        except json.JSONDecodeError as e:
            raise ConfigError(f"{path}: not valid JSON: {e}") from None
    if not isinstance(obj, dict):
        raise ConfigError(f"{path}: top level must be a JSON object")
    return obj


class ModelConfig:
    """Base of every architecture's typed configuration."""

    #: names under which config.json's ``architectures`` / ``model_type`` select this class
    architectures: tuple = ()

    @classmethod
    def from_dict(cls, obj: Dict[str, Any], where: str = "config.json"):
        cfg = cls(**parse_fields(cls, obj, where))
        cfg.validate(where)
        return cfg

    def validate(self, where: str) -> None:  # pragma: no cover - overridden
        pass

    def to_dict(self) -> Dict[str, Any]:
        """The JSON object that ``from_dict`` reads back to an equal configuration."""
        raise NotImplementedError
