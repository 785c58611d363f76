"""One registry from an architecture's name to its configuration class and model builder.

The reference hard-wires its single model
(/root/reference/include/runtime/gpt2_backend.h:13-14); here the class is chosen
by ``architectures[0]`` of config.json (``model_type`` as a fallback).
"""
from __future__ import annotations

import json
import os
from dataclasses import dataclass
from typing import Any, Callable, Dict, Optional, Type

from .base import ConfigError, ModelConfig


@dataclass
class Architecture:
    name: str
    config_cls: Type[ModelConfig]
    build: Callable[..., Any]           # (config, dtype, device) -> DecoderModel (weights not yet loaded)
    model_type: Optional[str] = None    # config.json "model_type" that also selects it


_ARCHITECTURES: Dict[str, Architecture] = {}


def register_architecture(name: str, config_cls: Type[ModelConfig], build: Callable[..., Any],
                          model_type: Optional[str] = None, replace: bool = False) -> None:
    if name in _ARCHITECTURES and not replace:
        raise ValueError(f"architecture '{name}' is already registered")
    _ARCHITECTURES[name] = Architecture(name, config_cls, build, model_type)


def registered_architectures():
    return sorted(_ARCHITECTURES)


def get_architecture(name: str) -> Architecture:
    if name not in _ARCHITECTURES:
        raise ConfigError(
            f"unknown architecture '{name}'; registered: {registered_architectures()}")
    return _ARCHITECTURES[name]


def architecture_of(d: Dict[str, Any]) -> Architecture:
    archs = d.get("architectures")
    if archs:
        return get_architecture(archs[0])
    mt = d.get("model_type")
    for a in _ARCHITECTURES.values():
        if mt is not None and a.model_type == mt:
            return a
    raise ConfigError(
        "config.json names no architecture ('architectures' or a known 'model_type'); "
        f"registered: {registered_architectures()}")


def load_config(model_dir: str) -> ModelConfig:
    path = os.path.join(model_dir, "config.json")
    if not os.path.isfile(path):
        raise ConfigError(f"{path}: no such file")
    with open(path) as f:
        try:
            d = json.load(f)
        except json.JSONDecodeError as e:
            raise ConfigError(f"{path}: not valid JSON ({e})") from None
    if not isinstance(d, dict):
        raise ConfigError(f"{path}: top level must be an object")
    return architecture_of(d).config_cls.from_dict(d)
