"""GPT-2 (GPT2LMHeadModel): which parts it is made of and what its tensors are called.

Tensor names are those of the GPT-2 checkpoint that the reference exports from
(/root/reference/scripts/export_weights.py:34-66): wte, wpe,
h.{i}.ln_1/attn.c_attn/attn.c_proj/ln_2/mlp.c_fc/mlp.c_proj, ln_f; an optional
``transformer.`` prefix is accepted by the loader.
"""
from __future__ import annotations

import dataclasses
import math
import re

import torch

from ..config.base import PartSpec
from ..config.gpt2 import GPT2Config
from ..config.registry import register_architecture
from ..parts import attention, block, embedding, mlp, norms  # noqa: F401  (register the parts)
from ..parts.base import NORMS, POSITIONS, build_part
from ..parts.embedding import TiedHead, TokenEmbedding
from .decoder import DecoderModel, build_layers

# Buffers of the attention mask that some checkpoints carry, and the tied head's alias.
IGNORED_TENSORS = (
    re.compile(r"^h\.\d+\.attn\.(bias|masked_bias)$"),
    re.compile(r"^lm_head\.weight$"),
)
OPTIONAL_PREFIXES = ("transformer.",)


def build_gpt2(config: GPT2Config, dtype: torch.dtype, device) -> DecoderModel:
    emb = TokenEmbedding(config.vocab_size, config.n_embd, "wte", dtype, device)
    pos = build_part(POSITIONS, PartSpec("learned_absolute", {
        "n_positions": config.n_positions, "size": config.n_embd, "name": "wpe"}), dtype, device,
        "position encoding")
    specs = config.layer_specs()
    # Residual projections are initialised with std 0.02 / sqrt(2 * n_layer) in random-weights mode.
    out_std = 0.02 / math.sqrt(2 * config.n_layer)
    specs = [dataclasses.replace(
        ls,
        mixer=PartSpec(ls.mixer.kind, {**ls.mixer.params, "out_init_std": out_std}),
        feed_forward=PartSpec(ls.feed_forward.kind, {**ls.feed_forward.params, "out_init_std": out_std}))
        for ls in specs]
    layers, prefixes = build_layers(specs, dtype, device)
    final_norm = build_part(NORMS, PartSpec("layernorm", {"size": config.n_embd,
                                                          "eps": config.layer_norm_epsilon}),
                            dtype, device, "norm")
    head = TiedHead(emb, dtype, device)
    model = DecoderModel(config, emb, pos, layers, prefixes, config.layer_order(), final_norm, "ln_f", head,
                         dtype, device)
    model.ignored_tensors = IGNORED_TENSORS
    model.optional_prefixes = OPTIONAL_PREFIXES
    return model


register_architecture("GPT2LMHeadModel", GPT2Config, build_gpt2, model_type="gpt2", replace=True)
