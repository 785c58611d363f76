"""Typed model configuration: what every architecture's config must provide.

A configuration is read from the architecture's own ``config.json`` keys and is
the only source of sizes and constants; parts receive them as parameters.

The engine needs three things from a configuration, whatever the architecture:

* ``layer_specs()``: for every layer, which block arrangement, mixer,
  feed-forward and norm it is built from, with their parameters;
* ``layer_order()``: the order in which layers run, as data (a layer may be
  named twice, and a call may read another call's cache);
* the sizes of the embedding, the final norm and the output head.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional, Tuple, Union


class ConfigError(ValueError):
    """A config.json that is missing a key, or holds a value the engine refuses."""


@dataclass(frozen=True)
class PartSpec:
    """Which registered part to build, and the parameters it is built with."""
    kind: str
    params: Dict[str, Any] = field(default_factory=dict)


@dataclass(frozen=True)
class LayerSpec:
    """One layer: a block arrangement over a mixer, a feed-forward and norms.

    ``mixer`` or ``feed_forward`` may be None: the arrangement then leaves that sub-layer (and its norm)
    out. ``norm`` is one spec, built once for every norm position of the block, or a tuple with one spec
    for each position (a layer whose norms differ in kind or constants)."""
    block: str                      # registered block arrangement, e.g. "pre_norm"
    mixer: Optional[PartSpec]
    feed_forward: Optional[PartSpec]
    norm: Union[PartSpec, Tuple[PartSpec, ...]]
    weight_prefix: str              # tensor-name prefix of this layer's weights
    norm_names: Tuple[str, ...] = ("ln_1", "ln_2")   # tensor names of the block's norms

    def norm_at(self, position: int) -> PartSpec:
        if isinstance(self.norm, PartSpec):
            return self.norm
        if position >= len(self.norm):
            raise ConfigError(f"layer '{self.weight_prefix}' gives {len(self.norm)} norms; its block asks for more")
        return self.norm[position]


@dataclass(frozen=True)
class LayerCall:
    """One entry of the execution order.

    ``layer``  index into the list of layers (may repeat);
    ``cache``  index of the cache this call uses; calls that share an index share
               keys/values (or state);
    ``write``  False when the call only reads a cache that an earlier call wrote.
    """
    layer: int
    cache: int
    write: bool = True


class ModelConfig:
    """Interface of a typed configuration. Subclasses are dataclasses."""

    architecture: str = ""

    # sizes every model needs
    vocab_size: int
    hidden_size: int

    @classmethod
    def from_dict(cls, d: Dict[str, Any]) -> "ModelConfig":
        raise NotImplementedError

    def to_dict(self) -> Dict[str, Any]:
        raise NotImplementedError

    def layer_specs(self) -> List[LayerSpec]:
        raise NotImplementedError

    def layer_order(self) -> List[LayerCall]:
        n = len(self.layer_specs())
        return [LayerCall(layer=i, cache=i, write=True) for i in range(n)]

    @property
    def max_positions(self) -> Optional[int]:
        """Longest sequence the architecture can hold, or None if unbounded."""
        return None

    @property
    def eos_token_id(self) -> Optional[int]:
        return None


def require(d: Dict[str, Any], key: str, typ, where: str = "config.json"):
    if key not in d or d[key] is None:
        raise ConfigError(f"{where}: required key '{key}' is missing")
    v = d[key]
    if typ is float and isinstance(v, int) and not isinstance(v, bool):
        v = float(v)
    if typ is int and isinstance(v, bool):
        raise ConfigError(f"{where}: key '{key}' must be an integer, got {v!r}")
    if not isinstance(v, typ):
        raise ConfigError(f"{where}: key '{key}' must be {typ.__name__}, got {v!r}")
    return v
