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
    """One layer: the arrangement (a registered block) and the parts it arranges, by role.

    Which roles a block has, and which kind of part fills each, is the block's own business
    (``Block.roles``); every block has a role "mixer", the part that may own a cache or state.
    """
    block: str                                         # arrangement of the parts, e.g. "prenorm"
    parts: Dict[str, PartSpec] = field(default_factory=dict)   # role -> part

    @classmethod
    def prenorm(cls, mixer: PartSpec, feed_forward: PartSpec, mixer_norm: PartSpec, ffn_norm: PartSpec) -> "LayerSpec":
        return cls("prenorm", {"mixer_norm": mixer_norm, "ffn_norm": ffn_norm, "mixer": mixer,
                               "feed_forward": feed_forward})

    @property
    def mixer(self) -> PartSpec:
        return self.parts["mixer"]


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
    # Checkpoint tensors the model does not read and the loader lets pass: names that end in one of
    # ``ignored_tensor_suffixes`` are exporters' buffers without learned values (no word is said);
    # a name in ``unused_tensors`` holds values this configuration has no use for (a warning).
    ignored_tensor_suffixes: Tuple[str, ...] = ()
    unused_tensors: Tuple[str, ...] = ()


@dataclass(frozen=True)
class CacheSpec:
    """What a mixer keeps per token in pages: ``key_width`` elements in the key pool and ``value_width`` in the
    value pool (for attention both are kv_heads * head_dim; a mixer with other needs says its own, and a width
    of 0 leaves that pool out).  How a page's elements are laid out is the mixer's own business.

    ``window`` None: every earlier position stays readable.  ``window`` W: a query at
    position p reads keys p-W+1..p only, so pages wholly before that may be given back.
    Caches with equal specs share a group: one block table, one pool of page numbers.
    """
    kv_heads: int
    head_dim: int
    window: Optional[int] = None
    key_width: Optional[int] = None        # elements per token; None: kv_heads * head_dim
    value_width: Optional[int] = None
    dtype: Optional[str] = None            # "float32" / "bfloat16" / "int32" of the pools; None: the mode's activation dtype

    def key_elements(self, page_size: int) -> int:
        return page_size * (self.kv_heads * self.head_dim if self.key_width is None else self.key_width)

    def value_elements(self, page_size: int) -> int:
        return page_size * (self.kv_heads * self.head_dim if self.value_width is None else self.value_width)


@dataclass(frozen=True)
class StateSpec:
    """Per-request state of fixed size that a mixer keeps in a slot (not in pages)."""
    shape: Tuple[int, ...]
    dtype: str = "float32"


# --------------------------------------------------------------------------- interfaces

class Part:
    """Base of every part.  ``runtime`` carries the device and the precision mode; what belongs
    to one engine (scratch buffers, page size, caches) arrives with every step's context."""

    graph_safe = False             # True if forward() launches only capturable device work
    launches_through_ops = False   # True if everything forward() puts on the stream goes through bitwise_amd.csrc.ops
                                   # (then a decode step may hold launches back to join them: ops.chain)

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


class Embedding(Part):
    def forward(self, ctx):
        """Token ids ``ctx.tokens`` -> the 32-bit residual stream [max_rows, width] (a buffer of
        the context's workspace; rows of negative tokens are zero)."""
        raise NotImplementedError


class Head(Part):
    def bind(self, tensors: Dict[str, Any], embedding: Optional[Embedding] = None) -> None:
        """As Part.bind; ``embedding`` is the model's embedding part (a tied head reads its table)."""

    def forward(self, ctx, x, norm, count: int):
        """x: ``count`` wanted rows of the 32-bit residual stream; runs ``norm`` and the
        projection; returns 32-bit logits [>= count, vocab]."""
        raise NotImplementedError


class Norm(Part):
    def forward(self, ctx, x):
        """x: [rows, width] 32-bit residual stream -> normed rows in the activation dtype."""
        raise NotImplementedError


class PositionEncoding(Part):
    """Owns its tables; mixers apply it through the kernels they call.

    What a mixer that rotates pairs of elements by a position's angles may rely on (the attention part refuses a
    position encoding that does not keep it):
    * ``rotary_dim``: how many leading elements of a head are rotated; even, at most the head size.  Element i is
      paired with element i + rotary_dim / 2 (the rotate-half layout).
    * ``tables()`` -> (cos, sin): two contiguous 32-bit tensors [positions, rotary_dim / 2] on the runtime's
      device, row p holding the cosines and sines of position p's angles; they do not move or change once made
      (captured graphs read them).
    * ``shared(params, runtime)``: the instance for these parameters (mixers of several layers may share one).
    What the angles are (base, scaling, stretching, learned) is the part's own business."""

    rotary_dim: int = 0

    def tables(self):
        raise NotImplementedError

    @classmethod
    def shared(cls, params, runtime):
        return cls(params, runtime)


class Mixer(Part):
    def cache_spec(self) -> Optional[CacheSpec]:
        return None

    def state_spec(self) -> Optional[StateSpec]:
        return None

    def page_sizes(self) -> Optional[Tuple[int, ...]]:
        """Page sizes (tokens) this mixer's kernels take for its paged cache; None: any."""
        return None

    @property
    def prefix_reusable(self) -> bool:
        """Whether a request may start behind cached pages of another request with the same first tokens: true
        if everything this mixer has computed for those tokens lies in its pages.  State in a slot does not."""
        return self.state_spec() is None

    @property
    def run_ahead_safe(self) -> bool:
        """Whether a decode step may be launched before the step before it is known to have been the last of a
        request (that request's row of the new step is then thrown away, after it has run).  By default a mixer
        with state of its own says no; one whose state may be advanced once more for a request that has ended
        (the slot is reset when it is taken again) overrides this."""
        return self.state_spec() is None

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
    def forward_with_norm(self, ctx, x, norm, residual) -> bool:
        """As Mixer.forward_with_norm."""
        return False

    def forward(self, ctx, h, residual) -> None:
        """h: normed rows; adds the feed-forward's output into ``residual`` in place."""
        raise NotImplementedError


class Block(Part):
    """The arrangement of a layer's parts around the residual stream.

    ``roles`` names the parts an arrangement has and the kind of each ("mixer", "feed_forward",
    "norm"), in the order their tensors are listed; the built parts become attributes of those
    names.  Every arrangement has a role "mixer"."""

    roles: Dict[str, str] = {}

    def __init__(self, parts: Dict[str, Part], runtime):
        super().__init__({}, runtime)
        missing = [r for r in self.roles if r not in parts]
        extra = [r for r in parts if r not in self.roles]
        if missing or extra:
            raise ValueError(f"block {type(self).__name__}: missing parts {missing}, unknown parts {extra}")
        self.parts = {role: parts[role] for role in self.roles}
        for role, part in self.parts.items():
            setattr(self, role, part)

    def forward(self, ctx, call, x) -> None:
        raise NotImplementedError


# --------------------------------------------------------------------------- registries

MIXERS: Dict[str, Type[Mixer]] = {}
FEED_FORWARDS: Dict[str, Type[FeedForward]] = {}
NORMS: Dict[str, Type[Norm]] = {}
POSITION_ENCODINGS: Dict[str, Type[PositionEncoding]] = {}
BLOCKS: Dict[str, Type[Block]] = {}
EMBEDDINGS: Dict[str, Type[Embedding]] = {}
HEADS: Dict[str, Type[Head]] = {}
# the registry of every kind of part a block's role may name
KINDS: Dict[str, Dict[str, type]] = {"mixer": MIXERS, "feed_forward": FEED_FORWARDS, "norm": NORMS}


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
register_embedding = _register(EMBEDDINGS, "embedding")
register_head = _register(HEADS, "head")


def lookup(table: Dict[str, type], what: str, name: str) -> type:
    try:
        return table[name]
    except KeyError:
        raise KeyError(f"unknown {what} '{name}'; registered: {sorted(table)}") from None
