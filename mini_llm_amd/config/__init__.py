"""Configurations and architectures, seen from Python: faces over the native registry
(csrc/engine/arch.cc). A configuration is a config.json dictionary; the architecture named in it
(``architectures[0]``, else ``model_type``) decides which keys it reads, which values it refuses and
which tensors a model of it expects. Presets are config.json files under ``config/presets``.
"""
from __future__ import annotations

import json
import os
from typing import Dict, List, Union

from .. import native

PRESETS_DIR = os.path.join(os.path.dirname(os.path.abspath(__file__)), "presets")


class ConfigError(ValueError):
    pass


def read_preset(name: str) -> dict:
    path = os.path.join(PRESETS_DIR, name + ".json")
    if not os.path.isfile(path):
        known = sorted(f[:-5] for f in os.listdir(PRESETS_DIR) if f.endswith(".json"))
        raise ConfigError(f"unknown preset '{name}' (known: {', '.join(known)})")
    with open(path) as f:
        return json.load(f)


def as_config(config: Union[str, dict]) -> dict:
    """A preset's name or a config.json dictionary."""
    return read_preset(config) if isinstance(config, str) else dict(config)


def registered_architectures() -> List[str]:
    lb = native.lib()
    return json.loads(native.text_of(lambda buf, cap: lb.mllm_registered_architectures(buf, cap)))


def load_plugin(path: str) -> None:
    """Loads a shared library whose initialisers register further parts and architectures with the engine."""
    try:
        native.check(native.lib().mllm_load_plugin(os.fsencode(path)))
    except native.EngineError as e:
        raise ConfigError(str(e)) from None


def describe_config(config: Union[str, dict]) -> Dict:
    """Checks a configuration as its architecture does and returns
    ``{"architecture": name, "tensors": [{"name", "shape", "role", "transpose", "mean", "std"}, ...]}``:
    the tensors a model of it expects. Raises ConfigError with the architecture's own message for a
    configuration that it refuses."""
    lb = native.lib()
    text = json.dumps(as_config(config)).encode()
    try:
        return json.loads(native.text_of(lambda buf, cap: lb.mllm_describe_config(text, buf, cap)))
    except native.EngineError as e:
        raise ConfigError(str(e)) from None
