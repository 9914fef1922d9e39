"""One registry from an architecture's name to its configuration class.

Detection follows the reference (src/arch/mod.rs:723-759): the first
registered architecture whose names match config.json's `architectures` entries or its
`model_type`; `arch=` forces one (the CLI's `--arch`,
src/main.rs:180-183).
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Dict, Mapping, Optional, Sequence, Tuple, Type

from .base import ArchConfig, ConfigError


@dataclass(frozen=True)
class Architecture:
    name: str                           # canonical name, e.g. "Lfm2ForCausalLM"
    aliases: Tuple[str, ...]            # model_type values and family names
    config_cls: Type[ArchConfig]


_REGISTRY: Dict[str, Architecture] = {}


def register_architecture(name: str, config_cls: Type[ArchConfig], aliases: Sequence[str] = ()) -> Architecture:
    arch = Architecture(name, tuple(aliases), config_cls)
    _REGISTRY[name] = arch
    return arch


def architectures() -> Tuple[Architecture, ...]:
    return tuple(_REGISTRY.values())


def find_architecture(cfg: Mapping[str, Any], arch: Optional[str] = None) -> Architecture:
    """The architecture a config.json names; `arch` overrides detection."""
    if arch is not None:
        for a in _REGISTRY.values():
            if arch == a.name or arch in a.aliases:
                return a
        raise ConfigError(f"unknown architecture {arch!r}; registered: {sorted(_REGISTRY)}")
    names = list(cfg.get("architectures") or [])
    model_type = cfg.get("model_type")
    for a in _REGISTRY.values():
        if any(n == a.name for n in names) or (model_type is not None and model_type in a.aliases):
            return a
    raise ConfigError(
        f"no architecture spec matches this checkpoint (architectures={names}, model_type={model_type!r}); "
        f"registered: {sorted(_REGISTRY)}")


def config_from_dict(cfg: Mapping[str, Any], tensors: Optional[Mapping[str, Sequence[int]]] = None,
                     arch: Optional[str] = None) -> ArchConfig:
    a = find_architecture(cfg, arch)
    return a.config_cls.from_dict(cfg, tensors)
