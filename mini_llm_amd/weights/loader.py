"""Loads a model's tensors from safetensors by name.

Every tensor the model's parts declare is looked up by its checkpoint name, checked
against the shape the configuration implies, converted and handed to its part:
matrices go to the compute dtype (bfloat16 or float32), vectors (biases, norm gains)
stay in 32-bit, integer tables become int32. One error lists everything that is
missing, unexpected or of the wrong shape.

The reference reads raw fp32 files by file name and only detects a short read
(/root/reference/src/model/gpt2_model.cu:32-70,115-173).
"""
from __future__ import annotations

import json
import os
from typing import Dict, Iterable, List, Tuple

import torch

from .safetensors_io import SafetensorsError, SafetensorsFile


class WeightsError(ValueError):
    """The checkpoint does not fit the model; the message lists every mismatch."""

    def __init__(self, message: str, missing=(), unexpected=(), wrong_shape=()):
        super().__init__(message)
        self.missing = list(missing)
        self.unexpected = list(unexpected)
        self.wrong_shape = list(wrong_shape)


def _checkpoint_files(model_dir: str) -> List[str]:
    index = os.path.join(model_dir, "model.safetensors.index.json")
    single = os.path.join(model_dir, "model.safetensors")
    if os.path.isfile(single):
        return [single]
    if os.path.isfile(index):
        with open(index) as f:
            shards = sorted(set(json.load(f)["weight_map"].values()))
        return [os.path.join(model_dir, s) for s in shards]
    raise WeightsError(f"{model_dir}: neither model.safetensors nor model.safetensors.index.json is there")


def load_weights(model, model_dir: str) -> None:
    files = [SafetensorsFile(p) for p in _checkpoint_files(model_dir)]
    try:
        _load(model, files, model_dir)
    finally:
        for f in files:
            f.close()


def _load(model, files: List[SafetensorsFile], where: str) -> None:
    ignored = getattr(model, "ignored_tensors", ())
    prefixes = getattr(model, "optional_prefixes", ())
    raw: Dict[str, Tuple[SafetensorsFile, str]] = {}
    for f in files:
        for name in f.names():
            if name in raw:
                raise WeightsError(f"{where}: tensor '{name}' appears in two files")
            raw[name] = (f, name)
    specs = {s.name: s for s in model.param_specs()}
    available: Dict[str, Tuple[SafetensorsFile, str]] = {}
    for name, src in raw.items():
        short = name
        for p in prefixes:
            if name.startswith(p) and name not in specs:
                short = name[len(p):]
                break
        if any(pat.match(short) for pat in ignored):
            continue
        available[short] = src

    missing = sorted(n for n in specs if n not in available)
    unexpected = sorted(n for n in available if n not in specs)
    wrong = []
    for n, s in specs.items():
        if n in available:
            f, stored = available[n]
            _, shape = f.info(stored)
            if tuple(shape) != tuple(s.shape):
                wrong.append((n, tuple(s.shape), tuple(shape)))
    if missing or unexpected or wrong:
        lines = [f"{where}: the checkpoint does not fit the model ({type(model.config).__name__})"]
        if missing:
            lines.append(f"  missing tensors ({len(missing)}): " + ", ".join(missing))
        if unexpected:
            lines.append(f"  unexpected tensors ({len(unexpected)}): " + ", ".join(unexpected))
        if wrong:
            lines.append(f"  wrong shapes ({len(wrong)}): " + "; ".join(
                f"{n}: expected {list(e)}, found {list(g)}" for n, e, g in wrong))
        raise WeightsError("\n".join(lines), missing, unexpected, wrong)

    for n, s in specs.items():
        f, stored = available[n]
        t = f.tensor(stored)
        if s.role == "matrix":
            if not t.is_floating_point():
                raise WeightsError(f"{where}: tensor '{n}' must be floating point, found {t.dtype}")
            if s.layout == "transpose":
                t = t.t()
            t = t.to(model.dtype).contiguous()
        elif s.role == "vector":
            if not t.is_floating_point():
                raise WeightsError(f"{where}: tensor '{n}' must be floating point, found {t.dtype}")
            t = t.to(torch.float32).contiguous()
        elif s.role == "table":
            t = t.to(torch.int32).contiguous()
        else:
            raise ValueError(f"unknown role '{s.role}' of tensor '{n}'")
        s.assign(t.to(model.device))
