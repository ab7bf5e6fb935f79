"""A model put together from parts according to a ModelSpec, and its forward pass over one
step's rows (the role of Runner::forward, src/model.cpp:267-322)."""

from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, List, Optional, Tuple

import torch

from ..csrc import ops
from ..parts import base
from ..parts.base import CacheSpec, LayerCall, ModelSpec, StateSpec, TensorSpec, lookup
from ..runtime import Runtime


@dataclass
class CallBinding:
    """One schedule entry made concrete: which layer runs, which cache group's block table covers
    its cache, and the cache tensors and state tensor it works on.  The model's own list
    (``AssembledModel.calls``) is the plan and carries no tensors; every cache storage makes
    bound copies of it (``CacheStorage.bindings``), so that engines on one model share nothing."""
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
        self.embedding = lookup(base.EMBEDDINGS, "embedding", spec.embedding.kind)(spec.embedding.params, runtime)
        self.layers: List[base.Block] = []
        for ls in spec.layers:
            block_cls = lookup(base.BLOCKS, "block", ls.block)
            if "mixer" not in block_cls.roles:
                raise ValueError(f"block '{ls.block}' has no role 'mixer'")
            parts = {}
            for role, ps in ls.parts.items():
                kind = block_cls.roles.get(role)
                if kind is None:
                    raise ValueError(f"block '{ls.block}' has no role '{role}'; its roles: {sorted(block_cls.roles)}")
                parts[role] = lookup(base.KINDS[kind], kind.replace("_", "-"), ps.kind)(ps.params, runtime)
            self.layers.append(block_cls(parts, runtime))
        self.final_norm = lookup(base.NORMS, "norm", spec.final_norm.kind)(spec.final_norm.params, runtime)
        self.lm_head = lookup(base.HEADS, "head", spec.lm_head.kind)(spec.lm_head.params, runtime)
        self._plan_caches(spec.schedule)
        every = [self.embedding, self.final_norm, self.lm_head] + [p for b in self.layers for p in (b, *b.parts.values())]
        self.graph_safe = all(getattr(p, "graph_safe", False) for p in every)
        # (a captured decode step may hold its launches back to join them only if none of them goes round ops)
        self.launches_through_ops = all(getattr(p, "launches_through_ops", False) for p in every)
        # each mixer's own word on what the engine may do around it (parts.base.Mixer)
        mixers = [self.layers[c.layer].mixer for c in spec.schedule]
        self.prefix_reusable = all(m.prefix_reusable for m in mixers)
        self.run_ahead_safe = all(m.run_ahead_safe for m in mixers)

    def check_page_size(self, page_size: int) -> None:
        """Refuse a page size that one of the mixers' kernels does not take."""
        for i, block in enumerate(self.layers):
            sizes = block.mixer.page_sizes()
            if sizes is not None and page_size not in sizes:
                raise ValueError(f"layer {i}: its mixer takes pages of {sorted(sizes)} tokens, not of {page_size}")

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
            for role, part in block.parts.items():
                yield ls.parts[role].prefix, part
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
                part.bind(mine, embedding=self.embedding)
            else:
                part.bind(mine)

    def weight_bytes(self) -> int:
        """Bytes of weights one decode step reads: every layer call's weights once, the final
        norm and the head (a tied head is the embedding table, read whole as the head)."""
        total = self.final_norm.weight_bytes() + self.lm_head.weight_bytes()
        for call in self.calls:
            total += sum(p.weight_bytes() for p in self.layers[call.layer].parts.values())
        return total

    # ------------------------------------------------------------------ forward
    def forward(self, ctx) -> Optional[torch.Tensor]:
        """Run the step's rows through every scheduled layer call; logits [wanted, vocab]
        (32-bit) for the wanted rows in row order, or None if nothing is wanted.  Everything
        that belongs to one engine comes with ``ctx``: its workspace (``ctx.ws``) and the layer
        calls bound to its caches and state (``ctx.calls``)."""
        if len(ctx.calls) != len(self.calls):
            raise ValueError("the step context carries no bindings for this model's layer calls")
        ws = ctx.ws
        x = self.embedding.forward(ctx)
        for call in ctx.calls:
            self.layers[call.layer].forward(ctx, call, x)
        count = ctx.num_wanted
        if count == 0:
            return None
        if getattr(ctx, "wants_every_row", False):
            last = x                                     # rows 0 .. count-1 are the wanted ones already
        else:
            last = ws.buffer("wanted_rows", self.spec.width, torch.float32, rows=ws.max_logit_rows)
            ops.gather_rows(x, ctx.want_rows, last, count)
        logits = self.lm_head.forward(ctx, last, self.final_norm, count)
        return logits[:count]
