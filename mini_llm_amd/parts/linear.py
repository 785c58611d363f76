"""A linear map with optional bias, the building block of mixers and feed-forwards.

The weight is held as ``[out, in]`` (k contiguous), the layout the matrix kernels
read. A checkpoint that stores ``[in, out]`` (GPT-2's Conv1D; the reference uses it
untransposed as x*W, /root/reference/scripts/export_weights.py:47-52 and
/root/reference/src/kernels/linear.cu:8-87) is transposed once when loaded.
"""
from __future__ import annotations

from typing import List, Optional, Tuple

import torch

from ..kernels import ops
from .base import ParamSpec


class Linear:
    def __init__(self, in_features: int, out_features: int, bias: bool, weight_layout: str,
                 dtype: torch.dtype, device, init_std: float = 0.02, bias_std: float = 0.02):
        if weight_layout not in ("in_out", "out_in"):
            raise ValueError(f"weight_layout must be 'in_out' or 'out_in', got {weight_layout!r}")
        if dtype == torch.bfloat16 and in_features % 8 != 0:
            raise ValueError(f"a bfloat16 linear map needs an input width that is a multiple of 8, got "
                             f"{in_features} (its kernels load 16 bytes at a time); use float32 for this size")
        self.in_features, self.out_features = in_features, out_features
        self.has_bias = bias
        self.weight_layout = weight_layout
        self.dtype, self.device = dtype, torch.device(device)
        self.init_std, self.bias_std = init_std, bias_std
        self.weight: Optional[torch.Tensor] = None      # [out, in], compute dtype
        self.bias: Optional[torch.Tensor] = None        # [out], fp32

    def param_specs(self, name: str) -> List[ParamSpec]:
        stored = ((self.in_features, self.out_features) if self.weight_layout == "in_out"
                  else (self.out_features, self.in_features))
        specs = [ParamSpec(name + ".weight", stored, "matrix", self._set_weight, (0.0, self.init_std),
                           "transpose" if self.weight_layout == "in_out" else "as_stored")]
        if self.has_bias:
            specs.append(ParamSpec(name + ".bias", (self.out_features,), "vector", self._set_bias,
                                   (0.0, self.bias_std)))
        return specs

    def _set_weight(self, t: torch.Tensor) -> None:
        assert t.shape == (self.out_features, self.in_features)
        self.weight = t

    def _set_bias(self, t: torch.Tensor) -> None:
        self.bias = t

    def __call__(self, a: torch.Tensor, out: torch.Tensor, epilogue: str = "store",
                 kv_scatter: Optional[tuple] = None) -> torch.Tensor:
        if kv_scatter is not None:
            return ops.linear(a, self.weight, self.bias, out, epilogue, kv_scatter=kv_scatter)
        return ops.linear(a, self.weight, self.bias, out, epilogue)
