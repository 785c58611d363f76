"""Random-weights mode: writes a model folder (config.json, model.safetensors) from a
configuration and a seed.

Every tensor the model's parts declare is drawn from a normal distribution with the
mean and standard deviation the part names (GPT-2: matrices and embeddings N(0, 0.02),
residual projections N(0, 0.02/sqrt(2 n_layer)), biases N(0, 0.02), norm gains
N(1, 0.1), norm biases N(0, 0.02)).

The generator is specified here completely, so that any program in any language draws
the same values: element ``i`` of the tensor called ``name`` under ``seed`` is

    key   = splitmix64(seed) ^ fnv1a64(name as UTF-8)
    a     = splitmix64(key + 2 i),  b = splitmix64(key + 2 i + 1)
    u1    = ((a >> 11) + 1) / 2^53      (in (0, 1]),   u2 = (b >> 11) / 2^53   (in [0, 1))
    z     = sqrt(-2 ln u1) * cos(2 pi u2)                  (Box-Muller, in float64)
    value = float32(mean + std * z)

with ``splitmix64(x)``: ``z = x + 0x9E3779B97F4A7C15; z = (z ^ z >> 30) * 0xBF58476D1CE4E5B9;
z = (z ^ z >> 27) * 0x94D049BB133111EB; return z ^ z >> 31`` (all modulo 2^64) and ``fnv1a64``
the 64-bit FNV-1a hash (offset basis 0xCBF29CE484222325, prime 0x100000001B3). A value
depends on (seed, name, index) only: not on the order of the tensors, on other tensors
or on the library that computes it. Matrices are stored in bfloat16 by default (round to
nearest even of the float32 value; vectors stay float32), so the 32-bit and the
bfloat16 path read identical values. The reference has no such mode.
"""
from __future__ import annotations

import json
import os
from typing import Dict, Union

import numpy as np
import torch

from ..config.base import ModelConfig
from ..config.registry import architecture_of
from .safetensors_io import save_file

_STORE = {"bfloat16": torch.bfloat16, "float32": torch.float32, "float16": torch.float16}
_M64 = (1 << 64) - 1


def splitmix64(x: int) -> int:
    z = (x + 0x9E3779B97F4A7C15) & _M64
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & _M64
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & _M64
    return z ^ (z >> 31)


def fnv1a64(data: bytes) -> int:
    h = 0xCBF29CE484222325
    for byte in data:
        h = ((h ^ byte) * 0x100000001B3) & _M64
    return h


def _splitmix64_np(x: np.ndarray) -> np.ndarray:
    z = x + np.uint64(0x9E3779B97F4A7C15)
    z = (z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
    z = (z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
    return z ^ (z >> np.uint64(31))


_PIECE = 1 << 18


def _piece(key: np.uint64, first: int, m: int, mean: float, std: float, out: np.ndarray) -> None:
    with np.errstate(over="ignore"):
        i = np.arange(first, first + m, dtype=np.uint64)
        a = _splitmix64_np(key + np.uint64(2) * i)
        b = _splitmix64_np(key + np.uint64(2) * i + np.uint64(1))
        u1 = ((a >> np.uint64(11)).astype(np.float64) + 1.0) * (1.0 / 9007199254740992.0)
        u2 = (b >> np.uint64(11)).astype(np.float64) * (1.0 / 9007199254740992.0)
        z = np.sqrt(-2.0 * np.log(u1)) * np.cos(2.0 * np.pi * u2)
        out[:] = (mean + std * z).astype(np.float32)


def normal_values(seed: int, name: str, n: int, mean: float, std: float, first: int = 0) -> np.ndarray:
    """Elements [first, first + n) of tensor ``name`` under ``seed`` as float32 (see the module text).
    Large tensors are computed in pieces by a few threads (every value depends on its index only)."""
    key = np.uint64(splitmix64(int(seed) & _M64) ^ fnv1a64(name.encode("utf-8")))
    out = np.empty(n, dtype=np.float32)
    pieces = [(lo, min(_PIECE, n - lo)) for lo in range(0, n, _PIECE)]
    if len(pieces) <= 2:
        for lo, m in pieces:
            _piece(key, first + lo, m, mean, std, out[lo:lo + m])
        return out
    from concurrent.futures import ThreadPoolExecutor
    workers = max(1, min(16, os.cpu_count() or 1))
    with ThreadPoolExecutor(max_workers=workers) as ex:
        list(ex.map(lambda p: _piece(key, first + p[0], p[1], mean, std, out[p[0]:p[0] + p[1]]), pieces))
    return out


def random_tensors(model, seed: int, weights_dtype: str = "bfloat16") -> Dict[str, torch.Tensor]:
    if weights_dtype not in _STORE:
        raise ValueError(f"weights_dtype must be one of {sorted(_STORE)}")
    out: Dict[str, torch.Tensor] = {}
    for s in model.param_specs():
        if s.role == "table":
            raise ValueError(f"tensor '{s.name}': integer tables have no random initialisation")
        mean, std = s.init
        n = 1
        for d in s.shape:
            n *= int(d)
        t = torch.from_numpy(normal_values(seed, s.name, n, mean, std)).reshape(tuple(s.shape))
        out[s.name] = t.to(_STORE[weights_dtype]) if s.role == "matrix" else t
    return out


def write_random_model(config: Union[ModelConfig, dict], out_dir: str, seed: int,
                       weights_dtype: str = "bfloat16") -> str:
    """Writes ``out_dir/config.json`` and ``out_dir/model.safetensors``; returns out_dir."""
    if isinstance(config, dict):
        arch = architecture_of(config)
        config = arch.config_cls.from_dict(config)
    else:
        arch = architecture_of({"architectures": [config.architecture]})
    model = arch.build(config, torch.float32, "cpu")      # parts only; no tensor is allocated
    tensors = random_tensors(model, seed, weights_dtype)
    os.makedirs(out_dir, exist_ok=True)
    d = config.to_dict()
    d.setdefault("architectures", [arch.name])
    d["torch_dtype"] = weights_dtype
    with open(os.path.join(out_dir, "config.json"), "w") as f:
        json.dump(d, f, indent=2)
    save_file(tensors, os.path.join(out_dir, "model.safetensors"),
              metadata={"format": "pt", "seed": str(seed)})
    return out_dir
