"""Model construction: config.json chooses the architecture, the checkpoint fills its parts."""
from __future__ import annotations

import torch

from ..config.registry import architecture_of, load_config
from . import gpt2  # noqa: F401  (registers GPT2LMHeadModel)

DTYPES = {"bfloat16": torch.bfloat16, "bf16": torch.bfloat16, "float32": torch.float32, "fp32": torch.float32}


def parse_dtype(dtype) -> torch.dtype:
    if isinstance(dtype, torch.dtype):
        if dtype not in (torch.bfloat16, torch.float32):
            raise ValueError(f"dtype must be bfloat16 or float32, got {dtype}")
        return dtype
    if dtype not in DTYPES:
        raise ValueError(f"dtype must be one of {sorted(DTYPES)}, got {dtype!r}")
    return DTYPES[dtype]


def load_model(model_dir: str, dtype="bfloat16", device="cuda:0"):
    """Builds the model that ``model_dir/config.json`` names and loads its weights."""
    from ..weights.loader import load_weights
    config = load_config(model_dir)
    arch = architecture_of({"architectures": [config.architecture]})
    model = arch.build(config, parse_dtype(dtype), device)
    load_weights(model, model_dir)
    return model
