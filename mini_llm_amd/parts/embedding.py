"""Token embedding, learned absolute positions, and the output head tied to the embedding."""
from __future__ import annotations

from typing import List, Optional

import torch

from ..kernels import ops
from .base import ParamSpec, Part, PositionEncoding, register_position


@register_position("learned_absolute")
class LearnedAbsolutePositions(PositionEncoding):
    """A table wpe[position, :] added where tokens are embedded
    (/root/reference/src/kernels/embedding.cu:23-43). Positions are absolute indices in
    the token's own sequence (/root/reference/src/model/gpt2_model.cu:379-386,466-469)."""

    def __init__(self, n_positions: int, size: int, name: str, dtype, device, init_std: float = 0.02):
        super().__init__(dtype, device)
        self.n_positions, self.size, self.name, self.init_std = n_positions, size, name, init_std
        self.table = None

    def param_specs(self, prefix: str) -> List[ParamSpec]:
        return [ParamSpec(prefix + self.name + ".weight", (self.n_positions, self.size), "matrix",
                          self._set, (0.0, self.init_std))]

    def _set(self, t):
        self.table = t

    @property
    def max_positions(self) -> Optional[int]:
        return self.n_positions


@register_position("none")
class NoPositions(PositionEncoding):
    def __init__(self, dtype, device):
        super().__init__(dtype, device)

    max_positions = None


class TokenEmbedding(Part):
    """x[t,:] = wte[id[t],:] (+ the position table's row, fused into the same kernel)."""

    def __init__(self, vocab_size: int, size: int, name: str, dtype, device, init_std: float = 0.02):
        super().__init__(dtype, device)
        self.vocab_size, self.size, self.name, self.init_std = vocab_size, size, name, init_std
        self.weight: Optional[torch.Tensor] = None     # [V, D]

    def param_specs(self, prefix: str) -> List[ParamSpec]:
        return [ParamSpec(prefix + self.name + ".weight", (self.vocab_size, self.size), "matrix",
                          self._set, (0.0, self.init_std))]

    def _set(self, t):
        self.weight = t

    def forward(self, ctx, position: Optional[PositionEncoding]) -> torch.Tensor:
        x = torch.empty((ctx.n_tokens, self.size), dtype=torch.float32, device=self.weight.device)
        table = position.table if position is not None else None
        ops.embed(ctx.token_ids, ctx.positions, self.weight, table, x)
        if position is not None and table is None:
            position.at_embedding(x, ctx)
        return x


class TiedHead(Part):
    """logits = h wte^T, fp32, no bias; the embedding matrix [V, D] is read in place as the
    [N, K] operand, so no transposed copy exists (the reference builds one:
    /root/reference/src/model/gpt2_model.cu:87-113,419-428)."""

    def __init__(self, embedding: TokenEmbedding, dtype, device):
        super().__init__(dtype, device)
        self.embedding = embedding

        self.weight_view = _HeadWeights(embedding)

    def forward(self, h: torch.Tensor) -> torch.Tensor:
        logits = torch.empty((h.shape[0], self.embedding.vocab_size), dtype=torch.float32, device=h.device)
        return ops.linear(h, self.embedding.weight, None, logits, "store_f32")

    def forward_normed(self, norm, x: torch.Tensor, rows: torch.Tensor) -> torch.Tensor:
        """logits of norm(x[rows]): lets the final norm fuse into the head's product."""
        logits = torch.empty((rows.numel(), self.embedding.vocab_size), dtype=torch.float32, device=x.device)
        return norm.linear(x, self.weight_view, logits, "store_f32", rows)


class _HeadWeights:
    """The tied head seen as a linear map without bias (weight = the embedding matrix)."""

    def __init__(self, embedding: TokenEmbedding):
        self._embedding = embedding
        self.bias = None

    @property
    def weight(self):
        return self._embedding.weight

    def __call__(self, a, out, epilogue="store"):
        return ops.linear(a, self.weight, None, out, epilogue)
