"""Dense feed-forward."""
from __future__ import annotations

from typing import Dict, List

import torch

from .base import FeedForward, NormedInput, ParamSpec, register_feed_forward
from .linear import Linear

_ACT_EPILOGUE = {"gelu_tanh": "gelu_tanh", "gelu_erf": "gelu_erf"}


@register_feed_forward("dense_mlp")
class DenseMLP(FeedForward):
    """x += act(h W_up + b_up) W_down + b_down, the activation fused into the first
    product and the residual add into the second
    (/root/reference/src/model/gpt2_model.cu:345-363). Activations: tanh-GELU
    (/root/reference/src/kernels/gelu.cu:7-9) and exact erf-GELU."""

    accepts_normed_input = True
    native_kind = "dense_mlp"

    def native_params(self):
        from ..kernels import ops
        return {"activation": self.activation, "dtype": ops._DT[self.dtype],
                "up.weight": self.up.weight, "up.bias": self.up.bias,
                "down.weight": self.down.weight, "down.bias": self.down.bias}

    def __init__(self, hidden_size: int, inner_size: int, activation: str, bias: bool, weight_layout: str,
                 names: Dict[str, str], dtype, device, init_std: float = 0.02, out_init_std: float = 0.02):
        super().__init__(dtype, device)
        if activation not in _ACT_EPILOGUE:
            raise ValueError(f"unknown activation '{activation}' (known: {sorted(_ACT_EPILOGUE)})")
        self.hidden_size, self.inner_size, self.activation = hidden_size, inner_size, activation
        self.names = dict(names)
        self.up = Linear(hidden_size, inner_size, bias, weight_layout, dtype, device, init_std)
        self.down = Linear(inner_size, hidden_size, bias, weight_layout, dtype, device, out_init_std)

    def param_specs(self, prefix: str) -> List[ParamSpec]:
        return self.up.param_specs(prefix + self.names["up"]) + self.down.param_specs(prefix + self.names["down"])

    def forward(self, h, ctx, x) -> None:
        inner = torch.empty((h.shape[0], self.inner_size), dtype=self.dtype, device=h.device)
        if isinstance(h, NormedInput):
            h.linear(self.up, inner, _ACT_EPILOGUE[self.activation])
        else:
            self.up(h, inner, _ACT_EPILOGUE[self.activation])
        self.down(inner, x, "add_residual")
