"""Base class of typed architecture configurations and helpers to read config.json."""
from __future__ import annotations

import json
import os
from typing import Any, Mapping

from .spec import ModelSpec


class ConfigError(ValueError):
    """A config.json that this architecture cannot run: the message names the key."""


def first(cfg: Mapping[str, Any], *keys: str, default: Any = None) -> Any:
    """The value of the first of `keys` that config.json holds (dotted keys descend into
    objects), else `default`: the precedence rule of the reference's config expressions
    (`first(cfg.a, cfg.b, ...)`, src/arch/expr.rs:723)."""
    for key in keys:
        node: Any = cfg
        for part in key.split("."):
            if isinstance(node, Mapping) and part in node and node[part] is not None:
                node = node[part]
            else:
                node = None
                break
        if node is not None:
            return node
    return default


def require(cfg: Mapping[str, Any], *keys: str) -> Any:
    value = first(cfg, *keys)
    if value is None:
        raise ConfigError(f"config.json lacks {' / '.join(keys)}")
    return value


class ArchConfig:
    """What every architecture's configuration offers to the rest of the framework."""

    architecture: str = ""

    @classmethod
    def from_dict(cls, cfg: Mapping[str, Any], tensors=None) -> "ArchConfig":
        """`tensors`, when given, is the checkpoint's table name -> shape; a configuration
        may use it for what config.json leaves open."""
        raise NotImplementedError

    @classmethod
    def from_json_file(cls, path: str) -> "ArchConfig":
        with open(path) as f:
            return cls.from_dict(json.load(f))

    def to_dict(self) -> dict:
        """config.json keys of this configuration (what the random-weights mode writes)."""
        raise NotImplementedError

    def model_spec(self) -> ModelSpec:
        raise NotImplementedError


def read_config_json(model_dir: str) -> dict:
    path = os.path.join(model_dir, "config.json")
    if not os.path.isfile(path):
        raise FileNotFoundError(f"{model_dir}: no config.json")
    with open(path) as f:
        return json.load(f)
