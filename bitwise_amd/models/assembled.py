"""A model put together from parts according to a ModelSpec, and its forward pass over one
step's rows (the role of Runner::forward, src/model.cpp:267-322)."""

from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, List, Optional, Tuple

import torch

from ..csrc import ops
from ..parts import base
from ..parts.base import CacheSpec, LayerCall, ModelSpec, StateSpec, TensorSpec, lookup
from ..parts.embedding import Embedding, LMHead
from ..runtime import Runtime


@dataclass
class CallBinding:
    """One schedule entry made concrete: which layer runs, which cache tensors and state
    tensor it works on, and which cache group's block table covers them."""
    index: int
    layer: int
    cache: int
    group: int                       # -1: the mixer keeps no paged cache
    cache_index: int                 # index of the cache inside its group's storage
    writes_cache: bool
    k_cache: Optional[torch.Tensor] = None
    v_cache: Optional[torch.Tensor] = None
    state: Optional[torch.Tensor] = None


class AssembledModel:
    def __init__(self, spec: ModelSpec, runtime: Runtime):
        self.spec, self.rt = spec, runtime
        self.embedding = Embedding(spec.embedding.params, runtime)
        self.layers: List[base.Block] = []
        for ls in spec.layers:
            mixer = lookup(base.MIXERS, "mixer", ls.mixer.kind)(ls.mixer.params, runtime)
            ff = lookup(base.FEED_FORWARDS, "feed-forward", ls.feed_forward.kind)(ls.feed_forward.params, runtime)
            n1 = lookup(base.NORMS, "norm", ls.mixer_norm.kind)(ls.mixer_norm.params, runtime)
            n2 = lookup(base.NORMS, "norm", ls.ffn_norm.kind)(ls.ffn_norm.params, runtime)
            self.layers.append(lookup(base.BLOCKS, "block", ls.block)(mixer, ff, n1, n2, runtime))
        self.final_norm = lookup(base.NORMS, "norm", spec.final_norm.kind)(spec.final_norm.params, runtime)
        self.lm_head = LMHead(spec.lm_head.params, runtime)
        self._plan_caches(spec.schedule)
        self.graph_safe = all(getattr(b.mixer, "graph_safe", False) and getattr(b.feed_forward, "graph_safe", False)
                              for b in self.layers)

    # ------------------------------------------------------------------ caches and state
    def _plan_caches(self, schedule: List[LayerCall]) -> None:
        """Sort the caches that the schedule names into groups of equal needs."""
        self.group_specs: List[CacheSpec] = []
        self.group_caches: List[List[int]] = []          # group -> cache numbers, in storage order
        cache_home: Dict[int, Tuple[int, int]] = {}       # cache number -> (group, index in group)
        self.calls: List[CallBinding] = []
        self.state_specs: Dict[int, StateSpec] = {}       # call index -> per-request state
        for idx, c in enumerate(schedule):
            if not 0 <= c.layer < len(self.layers):
                raise ValueError(f"schedule entry {idx} names layer {c.layer}, the model has {len(self.layers)}")
            mixer = self.layers[c.layer].mixer
            cs = mixer.cache_spec()
            group, cindex = -1, -1
            if cs is not None:
                if c.writes_cache:
                    if c.cache in cache_home:
                        raise ValueError(f"schedule entry {idx}: cache {c.cache} already has a writer")
                    if cs not in self.group_specs:
                        self.group_specs.append(cs)
                        self.group_caches.append([])
                    group = self.group_specs.index(cs)
                    cindex = len(self.group_caches[group])
                    self.group_caches[group].append(c.cache)
                    cache_home[c.cache] = (group, cindex)
                else:
                    if c.cache not in cache_home:
                        raise ValueError(f"schedule entry {idx} reads cache {c.cache} before any call wrote it")
                    group, cindex = cache_home[c.cache]
                    if self.group_specs[group] != cs:
                        raise ValueError(f"schedule entry {idx} reads cache {c.cache} of another shape")
            ss = mixer.state_spec()
            if ss is not None:
                self.state_specs[idx] = ss
            self.calls.append(CallBinding(idx, c.layer, c.cache, group, cindex, c.writes_cache))

    # ------------------------------------------------------------------ tensors
    def _parts_with_prefix(self):
        s = self.spec
        yield s.embedding.prefix, self.embedding
        for ls, block in zip(s.layers, self.layers):
            yield ls.mixer_norm.prefix, block.mixer_norm
            yield ls.ffn_norm.prefix, block.ffn_norm
            yield ls.mixer.prefix, block.mixer
            yield ls.feed_forward.prefix, block.feed_forward
        yield s.final_norm.prefix, self.final_norm
        yield s.lm_head.prefix, self.lm_head

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        """Every checkpoint tensor the model needs, by full name, in a fixed order."""
        out: Dict[str, TensorSpec] = {}
        for prefix, part in self._parts_with_prefix():
            for name, ts in part.tensors().items():
                full = prefix + name
                if full in out and out[full] != ts:
                    raise ValueError(f"tensor {full} is wanted with two shapes")
                out[full] = ts
        return out

    def bind_tensors(self, tensors: Dict[str, torch.Tensor]) -> None:
        for prefix, part in self._parts_with_prefix():
            mine = {name: tensors[prefix + name] for name in part.tensors()}
            if part is self.lm_head:
                part.bind(mine, self.embedding)
            else:
                part.bind(mine)

    def weight_bytes(self) -> int:
        """Bytes of weights one decode step reads: every layer call's weights once, the final
        norm and the head (a tied head is the embedding table, read whole as the head)."""
        total = self.final_norm.weight_bytes() + self.lm_head.weight_bytes()
        for call in self.calls:
            b = self.layers[call.layer]
            total += (b.mixer.weight_bytes() + b.feed_forward.weight_bytes() + b.mixer_norm.weight_bytes()
                      + b.ffn_norm.weight_bytes())
        return total

    # ------------------------------------------------------------------ forward
    def forward(self, ctx) -> Optional[torch.Tensor]:
        """Run the step's rows through every scheduled layer call; logits [wanted, vocab]
        (32-bit) for the wanted rows in row order, or None if nothing is wanted."""
        x = self.embedding.forward(ctx)
        for call in self.calls:
            self.layers[call.layer].forward(ctx, call, x)
        count = ctx.num_wanted
        if count == 0:
            return None
        if getattr(ctx, "wants_every_row", False):
            last = x                                     # rows 0 .. count-1 are the wanted ones already
        else:
            last = self.rt.buffer("wanted_rows", self.spec.width, torch.float32, rows=self.rt.max_logit_rows)
            ops.gather_rows(x, ctx.want_rows, last, count)
        logits = self.lm_head.forward_with_norm(ctx, last, self.final_norm, count)
        if logits is None:
            normed = self.final_norm.forward(ctx, last, out_name="final_normed", rows=count)
            logits = self.lm_head.forward(ctx, normed, count)
        return logits[:count]
