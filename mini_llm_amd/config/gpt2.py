"""GPT-2 configuration, read from the keys of a GPT-2 ``config.json``.

The reference fixes these sizes at compile time
(/root/reference/include/constants.h:5-10,25-28); here they are data.
"""
from __future__ import annotations

from dataclasses import dataclass, asdict
from typing import Any, Dict, List, Optional, Tuple

from .base import ConfigError, LayerSpec, ModelConfig, PartSpec, require

_ACTIVATIONS = {
    # config.json name -> activation of the feed-forward part
    "gelu_new": "gelu_tanh",
    "gelu_pytorch_tanh": "gelu_tanh",
    "gelu_fast": "gelu_tanh",
    "gelu": "gelu_erf",
}


@dataclass(frozen=True)
class GPT2Config(ModelConfig):
    vocab_size: int
    n_positions: int
    n_embd: int
    n_layer: int
    n_head: int
    layer_norm_epsilon: float
    n_inner: Optional[int] = None
    activation_function: str = "gelu_new"
    eos_token: Optional[int] = None
    bos_token: Optional[int] = None
    tie_word_embeddings: bool = True
    torch_dtype: Optional[str] = None
    architectures: Tuple[str, ...] = ("GPT2LMHeadModel",)

    architecture = "GPT2LMHeadModel"

    def __post_init__(self):
        for k in ("vocab_size", "n_positions", "n_embd", "n_layer", "n_head"):
            if getattr(self, k) <= 0:
                raise ConfigError(f"config.json: '{k}' must be positive, got {getattr(self, k)}")
        if self.n_embd % self.n_head != 0:
            raise ConfigError(
                f"config.json: n_embd={self.n_embd} is not divisible by n_head={self.n_head}")
        if self.n_inner is not None and self.n_inner <= 0:
            raise ConfigError(f"config.json: n_inner must be positive, got {self.n_inner}")
        if self.activation_function not in _ACTIVATIONS:
            raise ConfigError(
                f"config.json: activation_function '{self.activation_function}' is not supported "
                f"(known: {sorted(_ACTIVATIONS)})")
        if not (self.layer_norm_epsilon > 0):
            raise ConfigError("config.json: layer_norm_epsilon must be positive")
        if not self.tie_word_embeddings:
            raise ConfigError("config.json: tie_word_embeddings=false (an untied head) is not supported")

    # ---- derived sizes -------------------------------------------------
    @property
    def hidden_size(self) -> int:
        return self.n_embd

    @property
    def head_dim(self) -> int:
        return self.n_embd // self.n_head

    @property
    def inner_dim(self) -> int:
        # GPT-2's rule: a missing n_inner means four times the width.
        return self.n_inner if self.n_inner is not None else 4 * self.n_embd

    @property
    def max_positions(self) -> Optional[int]:
        return self.n_positions

    @property
    def eos_token_id(self) -> Optional[int]:
        return self.eos_token

    # ---- (de)serialisation ----------------------------------------------
    @classmethod
    def from_dict(cls, d: Dict[str, Any]) -> "GPT2Config":
        refused = {
            "scale_attn_by_inverse_layer_idx": True,
            "reorder_and_upcast_attn": True,
            "add_cross_attention": True,
        }
        for k, bad in refused.items():
            if d.get(k, False) == bad:
                raise ConfigError(f"config.json: {k}={bad} is not supported")
        if d.get("scale_attn_weights", True) is False:
            raise ConfigError("config.json: scale_attn_weights=false is not supported")
        n_inner = d.get("n_inner")
        if n_inner is not None and (isinstance(n_inner, bool) or not isinstance(n_inner, int)):
            raise ConfigError(f"config.json: n_inner must be an integer or null, got {n_inner!r}")
        archs = d.get("architectures") or ["GPT2LMHeadModel"]
        return cls(
            vocab_size=require(d, "vocab_size", int),
            n_positions=require(d, "n_positions", int),
            n_embd=require(d, "n_embd", int),
            n_layer=require(d, "n_layer", int),
            n_head=require(d, "n_head", int),
            layer_norm_epsilon=require(d, "layer_norm_epsilon", float),
            n_inner=n_inner,
            activation_function=d.get("activation_function", "gelu_new"),
            eos_token=d.get("eos_token_id"),
            bos_token=d.get("bos_token_id"),
            tie_word_embeddings=bool(d.get("tie_word_embeddings", True)),
            torch_dtype=d.get("torch_dtype"),
            architectures=tuple(archs),
        )

    def to_dict(self) -> Dict[str, Any]:
        d = asdict(self)
        d["eos_token_id"] = d.pop("eos_token")
        d["bos_token_id"] = d.pop("bos_token")
        d["architectures"] = list(self.architectures)
        d["model_type"] = "gpt2"
        return d

    # ---- what the layers are made of ---------------------------------------
    def layer_specs(self) -> List[LayerSpec]:
        norm = PartSpec("layernorm", {"size": self.n_embd, "eps": self.layer_norm_epsilon})
        mixer = PartSpec("causal_attention", {
            "hidden_size": self.n_embd,
            "n_heads": self.n_head,
            "n_kv_heads": self.n_head,
            "head_dim": self.head_dim,
            "scale": self.head_dim ** -0.5,
            "window": None,
            "bias": True,
            "weight_layout": "in_out",      # Conv1D: stored [in, out]
            "names": {"qkv": "attn.c_attn", "out": "attn.c_proj"},
        })
        ff = PartSpec("dense_mlp", {
            "hidden_size": self.n_embd,
            "inner_size": self.inner_dim,
            "activation": _ACTIVATIONS[self.activation_function],
            "bias": True,
            "weight_layout": "in_out",
            "names": {"up": "mlp.c_fc", "down": "mlp.c_proj"},
        })
        return [
            LayerSpec(block="pre_norm", mixer=mixer, feed_forward=ff, norm=norm,
                      weight_prefix=f"h.{i}.")
            for i in range(self.n_layer)
        ]
