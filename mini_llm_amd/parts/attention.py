"""Causal self-attention over the paged cache."""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from ..cache.manager import KVCacheSpec, KVCacheView
from ..kernels import ops
from .base import Mixer, NormedInput, ParamSpec, PositionEncoding, register_mixer
from .linear import Linear


@register_mixer("causal_attention")
class CausalSelfAttention(Mixer):
    """qkv = h W_qkv + b; keys/values of the step's tokens go to the pages; every query
    attends causally (optionally within a window) to its sequence's keys in the pages;
    x += concat_heads(attn) W_out + b.

    Reference: /root/reference/src/model/gpt2_model.cu:289-334 (QKV, page write, attention,
    output projection with the residual add fused into the product).
    Column layout of qkv: queries [0, H*dh), keys [H*dh, H*dh + Hkv*dh), values after
    them; head h at h*dh (/root/reference/src/kernels/prefill/append_kv.cu:31-33).
    """

    accepts_normed_input = True
    native_kind = "causal_attention"

    def native_params(self):
        return {"n_heads": self.n_heads, "n_kv_heads": self.n_kv_heads, "head_dim": self.head_dim,
                "scale": self.scale, "window": self.window, "dtype": ops._DT[self.dtype],
                "qkv.weight": self.qkv.weight, "qkv.bias": self.qkv.bias,
                "out.weight": self.out.weight, "out.bias": self.out.bias}

    def __init__(self, hidden_size: int, n_heads: int, n_kv_heads: int, head_dim: int, scale: float,
                 window: Optional[int], bias: bool, weight_layout: str, names: Dict[str, str],
                 dtype, device, position: Optional[PositionEncoding] = None,
                 init_std: float = 0.02, out_init_std: float = 0.02):
        super().__init__(dtype, device)
        if n_heads % n_kv_heads != 0:
            raise ValueError(f"n_heads={n_heads} is not a multiple of n_kv_heads={n_kv_heads}")
        if head_dim % 16 != 0 or head_dim > 256:
            raise ValueError(f"head_dim={head_dim} is not supported (multiples of 16 up to 256)")
        self.hidden_size, self.n_heads, self.n_kv_heads, self.head_dim = hidden_size, n_heads, n_kv_heads, head_dim
        self.scale = float(scale)
        self.window = int(window or 0)
        self.q_dim, self.kv_dim = n_heads * head_dim, n_kv_heads * head_dim
        self.names = dict(names)
        self.position = position
        self.qkv = Linear(hidden_size, self.q_dim + 2 * self.kv_dim, bias, weight_layout, dtype, device, init_std)
        self.out = Linear(self.q_dim, hidden_size, bias, weight_layout, dtype, device, out_init_std)

    def param_specs(self, prefix: str) -> List[ParamSpec]:
        return self.qkv.param_specs(prefix + self.names["qkv"]) + self.out.param_specs(prefix + self.names["out"])

    def cache_spec(self):
        return KVCacheSpec(self.n_kv_heads, self.head_dim, self.window)

    def forward(self, h, ctx, cache_view: KVCacheView, x, write: bool = True) -> None:
        T = h.shape[0]
        g = cache_view.group
        qkv = torch.empty((T, self.q_dim + 2 * self.kv_dim), dtype=self.dtype, device=h.device)
        # Prompt portions: the QKV product is asked to put the new keys and values into the pages
        # (how is the linear map's business), unless a position encoding still has to turn them.
        # Single tokens: the attention kernel writes them.
        scatter = write and self.position is None and ctx.max_q_len > 1
        opts = {"kv_scatter": (ctx.slots[g], cache_view.k_pages, cache_view.v_pages, self.q_dim)} if scatter else {}
        if isinstance(h, NormedInput):
            h.linear(self.qkv, qkv, "store", **opts)
        else:
            self.qkv(h, qkv, "store", **opts)
        if self.position is not None:
            self.position.in_mixer(qkv, self, ctx)
        append = (self.q_dim, self.q_dim + self.kv_dim, ctx.slots[g]) if write and not scatter else None
        attn = torch.empty((T, self.q_dim), dtype=self.dtype, device=h.device)
        # (the result may come back unmerged, as the states of several workgroups per token and head:
        # the output projection takes either)
        attn = ops.paged_attention(qkv, 0, self.n_heads, self.n_kv_heads, self.head_dim,
                                   cache_view.k_pages, cache_view.v_pages, cache_view.page_size,
                                   ctx.block_tables[g], ctx.token_seq, ctx.positions, self.scale, self.window, attn,
                                   cu_q=ctx.cu_q, ctx_len=ctx.ctx_len, max_q_len=ctx.max_q_len,
                                   max_ctx_len=ctx.max_ctx_len, append=append, n_single=ctx.n_single,
                                   may_split=True)
        self.out(attn, x, "add_residual")
