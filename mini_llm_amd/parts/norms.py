"""Normalisation parts."""
from __future__ import annotations

from typing import List, Optional

import torch

from ..kernels import ops
from .base import Norm, ParamSpec, register_norm


@register_norm("layernorm")
class LayerNorm(Norm):
    """y = (x - mean) * rsqrt(var + eps) * gamma + beta over the last dimension, biased
    variance, statistics in fp32 (/root/reference/src/kernels/layernorm.cu:32-49).
    Input: the fp32 stream. Output: the compute dtype."""

    native_kind = "layernorm"

    def __init__(self, size: int, eps: float, dtype, device, bias: bool = True):
        super().__init__(dtype, device)
        self.size, self.eps, self.has_bias = int(size), float(eps), bool(bias)
        self.gamma: Optional[torch.Tensor] = None
        self.beta: Optional[torch.Tensor] = None

    def param_specs(self, prefix: str) -> List[ParamSpec]:
        specs = [ParamSpec(prefix + ".weight", (self.size,), "vector", self._set_gamma, (1.0, 0.1))]
        if self.has_bias:
            specs.append(ParamSpec(prefix + ".bias", (self.size,), "vector", self._set_beta, (0.0, 0.02)))
        return specs

    def native_params(self):
        return {"size": self.size, "eps": self.eps, "dtype": ops._DT[self.dtype], "gamma": self.gamma, "beta": self.beta}

    def _set_gamma(self, t):
        self.gamma = t

    def _set_beta(self, t):
        self.beta = t

    def linear(self, x: torch.Tensor, lin, out: torch.Tensor, epilogue: str = "store",
               rows: Optional[torch.Tensor] = None, **linear_options) -> torch.Tensor:
        """out = epilogue(lin(norm(x[rows]))): the norm fused into the product where the kernels allow it."""
        return ops.ln_linear(x, self.gamma, self.beta, self.eps, lin.weight, lin.bias, out, epilogue, rows,
                             **linear_options)

    def forward(self, x: torch.Tensor, rows: Optional[torch.Tensor] = None) -> torch.Tensor:
        n = rows.numel() if rows is not None else x.shape[0]
        out = torch.empty((n, self.size), dtype=self.dtype, device=x.device)
        return ops.layernorm(x, self.gamma, self.beta, self.eps, out, rows)
