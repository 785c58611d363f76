"""Random-weights mode: writes a model folder (config.json, model.safetensors) from a
configuration and a seed.

Every tensor the model's parts declare is drawn from a normal distribution with the
mean and standard deviation the part names (GPT-2: matrices and embeddings N(0, 0.02),
residual projections N(0, 0.02/sqrt(2 n_layer)), biases N(0, 0.02), norm gains
N(1, 0.1), norm biases N(0, 0.02)), in the order the model lists them, from one
``torch.Generator`` seeded with ``seed``. Matrices are stored in bfloat16 by default
(vectors in float32), so the 32-bit and the bfloat16 path read identical values.
The reference has no such mode.
"""
from __future__ import annotations

import json
import os
from typing import Dict, Union

import torch

from ..config.base import ModelConfig
from ..config.registry import architecture_of
from .safetensors_io import save_file

_STORE = {"bfloat16": torch.bfloat16, "float32": torch.float32, "float16": torch.float16}


def random_tensors(model, seed: int, weights_dtype: str = "bfloat16") -> Dict[str, torch.Tensor]:
    if weights_dtype not in _STORE:
        raise ValueError(f"weights_dtype must be one of {sorted(_STORE)}")
    gen = torch.Generator(device="cpu")
    gen.manual_seed(int(seed))
    out: Dict[str, torch.Tensor] = {}
    for s in model.param_specs():
        if s.role == "table":
            raise ValueError(f"tensor '{s.name}': integer tables have no random initialisation")
        mean, std = s.init
        t = torch.empty(s.shape, dtype=torch.float32).normal_(mean, std, generator=gen)
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
