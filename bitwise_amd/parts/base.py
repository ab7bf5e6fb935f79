"""What a model is made of: specs (plain data), part interfaces and the part registries.

A model is described by a ``ModelSpec``: a list of layers, each naming its mixer,
feed-forward and norms by registry key with their sizes as parameters, and a
*schedule*, the list of layer calls in the order they run.  A schedule entry names a
layer (so a layer may run twice) and the cache it reads (so a layer may read the
cache another call wrote).  No part knows which model it is in: everything it needs
arrives through its parameters, its tensors and the per-step ``StepContext``.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Callable, Dict, List, Optional, Tuple, Type


# --------------------------------------------------------------------------- specs

@dataclass(frozen=True)
class TensorSpec:
    """One checkpoint tensor a part needs: its shape and what kind of values it holds.

    kind: "linear" / "embedding" (random init N(0, sigma)), "norm" (1 + N(0, 0.1)) or
    "int" (integer table, kept as int32).
    """
    shape: Tuple[int, ...]
    kind: str = "linear"


@dataclass
class PartSpec:
    kind: str                      # registry key of the part's class
    params: Dict[str, Any] = field(default_factory=dict)   # sizes and constants
    prefix: str = ""               # prefix of the part's tensor names in the checkpoint


@dataclass
class LayerSpec:
    block: str                     # arrangement of the parts, e.g. "prenorm"
    mixer: PartSpec
    feed_forward: PartSpec
    mixer_norm: PartSpec
    ffn_norm: PartSpec


@dataclass(frozen=True)
class LayerCall:
    """One entry of the schedule: run ``layer``, with cache number ``cache``.

    ``writes_cache`` False means the call only reads a cache that an earlier call of
    the same step wrote (its own keys and values are not stored).
    """
    layer: int
    cache: int
    writes_cache: bool = True


@dataclass
class ModelSpec:
    architecture: str
    vocab_size: int
    width: int
    embedding: PartSpec
    layers: List[LayerSpec]
    schedule: List[LayerCall]
    final_norm: PartSpec
    lm_head: PartSpec
    max_positions: int
    bos_token_id: int = -1
    eos_token_id: int = -1


@dataclass(frozen=True)
class CacheSpec:
    """What a mixer keeps per token: keys and values in pages.

    ``window`` None: every earlier position stays readable.  ``window`` W: a query at
    position p reads keys p-W+1..p only, so pages wholly before that may be given back.
    """
    kv_heads: int
    head_dim: int
    window: Optional[int] = None


@dataclass(frozen=True)
class StateSpec:
    """Per-request state of fixed size that a mixer keeps in a slot (not in pages)."""
    shape: Tuple[int, ...]
    dtype: str = "float32"


# --------------------------------------------------------------------------- interfaces

class Part:
    """Base of every part.  ``runtime`` carries device, precision mode and kernels."""

    def __init__(self, params: Dict[str, Any], runtime: "Any"):
        self.params = dict(params)
        self.rt = runtime

    def tensors(self) -> Dict[str, TensorSpec]:
        """Checkpoint tensors by name relative to the part's prefix."""
        return {}

    def bind(self, tensors: Dict[str, Any]) -> None:
        """Take the loaded tensors (same keys as ``tensors()``), already on the device."""

    def weight_bytes(self) -> int:
        """Bytes a decode step reads from this part's weights (for the roofline)."""
        return 0


class Norm(Part):
    def forward(self, ctx, x):
        """x: [rows, width] 32-bit residual stream -> normed rows in the activation dtype."""
        raise NotImplementedError


class PositionEncoding(Part):
    """Owns its table(s); mixers apply it through the kernels they call."""


class Mixer(Part):
    graph_safe = False             # True if forward() launches only capturable device work

    def cache_spec(self) -> Optional[CacheSpec]:
        return None

    def state_spec(self) -> Optional[StateSpec]:
        return None

    def forward(self, ctx, call, h, residual) -> None:
        """h: normed rows [rows, width]; adds the mixer's output into ``residual`` in place.

        ``call`` is a ``CallBinding``: the cache tensors, the cache group's block table
        name and the state tensor that belong to this call of the layer.
        """
        raise NotImplementedError

    def forward_with_norm(self, ctx, call, x, norm, residual) -> bool:
        """Optional: run ``norm`` and the mixer as fused kernels on the un-normed rows ``x``.
        Return False (and do nothing) if this step cannot be fused; the block then calls the
        norm and ``forward`` one after the other.  The result must be the same bits."""
        return False


class FeedForward(Part):
    graph_safe = False

    def forward_with_norm(self, ctx, x, norm, residual) -> bool:
        """As Mixer.forward_with_norm."""
        return False

    def forward(self, ctx, h, residual) -> None:
        """h: normed rows; adds the feed-forward's output into ``residual`` in place."""
        raise NotImplementedError


class Block(Part):
    """The arrangement of mixer, feed-forward and norms around the residual stream."""

    def __init__(self, mixer: Mixer, feed_forward: FeedForward, mixer_norm: Norm, ffn_norm: Norm, runtime):
        super().__init__({}, runtime)
        self.mixer, self.feed_forward, self.mixer_norm, self.ffn_norm = mixer, feed_forward, mixer_norm, ffn_norm

    def forward(self, ctx, call, x) -> None:
        raise NotImplementedError


# --------------------------------------------------------------------------- registries

MIXERS: Dict[str, Type[Mixer]] = {}
FEED_FORWARDS: Dict[str, Type[FeedForward]] = {}
NORMS: Dict[str, Type[Norm]] = {}
POSITION_ENCODINGS: Dict[str, Type[PositionEncoding]] = {}
BLOCKS: Dict[str, Type[Block]] = {}


def _register(table: Dict[str, type], what: str) -> Callable[[str], Callable[[type], type]]:
    def by_name(name: str):
        def deco(cls):
            if name in table and table[name] is not cls:
                raise ValueError(f"{what} '{name}' is already registered")
            table[name] = cls
            return cls
        return deco
    return by_name


register_mixer = _register(MIXERS, "mixer")
register_feed_forward = _register(FEED_FORWARDS, "feed-forward")
register_norm = _register(NORMS, "norm")
register_position_encoding = _register(POSITION_ENCODINGS, "position encoding")
register_block = _register(BLOCKS, "block")


def lookup(table: Dict[str, type], what: str, name: str) -> type:
    try:
        return table[name]
    except KeyError:
        raise KeyError(f"unknown {what} '{name}'; registered: {sorted(table)}") from None
