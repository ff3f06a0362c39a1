"""One registry from an architecture's name (config.json "architectures"[0]) to
its configuration class and its model builder.

The reference has no registry: its engine assumes Llama and never reads
`architectures` (src/weights.cpp:55-121). Everything in this framework that
needs a model goes through `resolve`.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Callable, Mapping

from .base import ConfigError, read_model_json


@dataclass(frozen=True)
class Architecture:
    name: str
    parse_config: Callable[..., Any]     # (config dict, generation dict | None, architecture=name) -> config
    build_model: Callable[..., Any]      # (config) -> DecoderModel, its tensors not yet loaded


_ARCHITECTURES: dict[str, Architecture] = {}


def register_architecture(name: str, parse_config: Callable[..., Any],
                          build_model: Callable[..., Any], replace: bool = False) -> None:
    if name in _ARCHITECTURES and not replace:
        raise ValueError(f"architecture {name!r} is already registered")
    _ARCHITECTURES[name] = Architecture(name, parse_config, build_model)


def known_architectures() -> list[str]:
    return sorted(_ARCHITECTURES)


def architecture_name(cfg: Mapping[str, Any]) -> str:
    archs = cfg.get("architectures")
    if not isinstance(archs, list) or not archs or not isinstance(archs[0], str):
        raise ConfigError("config.json: key 'architectures' must be a non-empty list of names; "
                          f"known architectures: {known_architectures()}")
    return archs[0]


def resolve(name: str) -> Architecture:
    if name not in _ARCHITECTURES:
        raise ConfigError(f"unknown architecture {name!r}; known architectures: {known_architectures()}")
    return _ARCHITECTURES[name]


def parse_config(cfg: Mapping[str, Any], generation_cfg: Mapping[str, Any] | None = None) -> Any:
    """config.json contents -> the typed configuration of its architecture."""
    name = architecture_name(cfg)
    return resolve(name).parse_config(cfg, generation_cfg, architecture=name)


def load_config(model_dir: str) -> Any:
    cfg, gen = read_model_json(model_dir)
    return parse_config(cfg, gen)
