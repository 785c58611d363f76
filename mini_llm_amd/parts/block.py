"""Arrangements of a mixer, a feed-forward and norms in one layer."""
from __future__ import annotations

from typing import List, Sequence

from .base import Block, FeedForward, Mixer, Norm, NormedInput, ParamSpec, register_block


@register_block("pre_norm")
class PreNormBlock(Block):
    """x += mixer(norm1(x)); x += feed_forward(norm2(x)): the norm stands before each
    sub-layer, on the residual stream (/root/reference/src/model/gpt2_model.cu:279-363).
    A layer built without a mixer or without a feed-forward leaves that half, and its norm, out."""

    n_norms = 2

    @property
    def native_kind(self):
        return "pre_norm" if self.mixer is not None and self.feed_forward is not None else None

    def native_norms(self):
        return [self.norm1, self.norm2]

    def __init__(self, mixer: Mixer, feed_forward: FeedForward, norms: Sequence[Norm],
                 norm_names: Sequence[str], dtype, device):
        super().__init__(dtype, device)
        if len(norms) != 2 or len(norm_names) != 2:
            raise ValueError("a pre-norm block has two norms")
        self.mixer, self.feed_forward = mixer, feed_forward
        self.norm1, self.norm2 = norms
        self.norm_names = tuple(norm_names)

    def param_specs(self, prefix: str) -> List[ParamSpec]:
        specs: List[ParamSpec] = []
        if self.mixer is not None:
            specs += self.norm1.param_specs(prefix + self.norm_names[0]) + self.mixer.param_specs(prefix)
        if self.feed_forward is not None:
            specs += self.norm2.param_specs(prefix + self.norm_names[1]) + self.feed_forward.param_specs(prefix)
        return specs

    def cache_spec(self):
        return None if self.mixer is None else self.mixer.cache_spec()

    def forward(self, x, ctx, cache_view, write: bool = True) -> None:
        if self.mixer is not None:
            h = NormedInput(self.norm1, x) if self.mixer.accepts_normed_input else self.norm1.forward(x)
            self.mixer.forward(h, ctx, cache_view, x, write)
        if self.feed_forward is not None:
            h = NormedInput(self.norm2, x) if self.feed_forward.accepts_normed_input else self.norm2.forward(x)
            self.feed_forward.forward(h, ctx, x)
