"""Model folders, seen from Python: faces over the native loader and generator (csrc/engine/weights.cc).

A model folder holds config.json and model.safetensors (or the shards of model.safetensors.index.json).
"""
from __future__ import annotations

import ctypes
import json
import os
from typing import Tuple, Union

import numpy as np

from .. import native
from ..config import as_config


class WeightsError(ValueError):
    pass


def write_random_model(config: Union[str, dict], out_dir: str, seed: int, weights_dtype: str = "bfloat16") -> str:
    """Writes config.json and model.safetensors with random weights from the specified generator: value i
    of tensor ``name`` depends on (seed, name, i) only. Returns ``out_dir``."""
    os.makedirs(out_dir, exist_ok=True)
    try:
        native.check(native.lib().mllm_write_random_model(json.dumps(as_config(config)).encode(), int(seed),
                                                          os.fsencode(out_dir), weights_dtype.encode()))
    except native.EngineError as e:
        raise WeightsError(str(e)) from None
    return out_dir


def check_model_dir(model_dir: str) -> Tuple[str, int, int]:
    """Checks a folder's configuration and tensor names and shapes against its architecture without
    touching a GPU. Returns (architecture, tensors, parameters); ONE WeightsError lists every missing,
    unexpected and wrong-shaped tensor."""
    buf = ctypes.create_string_buffer(1024)
    if native.lib().mllm_check_model_dir(os.fsencode(model_dir), buf, 1024) != 0:
        raise WeightsError(native.last_error())
    arch, n_tensors, n_params = buf.value.decode().rsplit(" ", 2)
    return arch, int(n_tensors), int(n_params)


def normal_values(seed: int, name: str, first: int, n: int, mean: float = 0.0, std: float = 1.0) -> np.ndarray:
    """Values ``first .. first + n`` of the random generator for tensor ``name`` under ``seed`` (float32)."""
    out = np.empty(n, dtype=np.float32)
    native.check(native.lib().mllm_normal_values(int(seed), name.encode(), int(first), int(n), float(mean), float(std),
                                                 out.ctypes.data))
    return out
