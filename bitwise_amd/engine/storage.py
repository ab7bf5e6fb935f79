"""Device memory behind the cache manager: for every cache group one pool of key pages and
one of value pages per cache, and for every layer call with per-request state one tensor
with a row per slot (the role of KVPool, src/model.h:64-76; zero-initialised as
src/model.cpp:246-247).  Page p of a group is the same page number in all of its caches.
A storage belongs to one engine: it binds copies of the model's layer calls to its own
tensors and leaves the model untouched, so any number of storages may serve one model.
"""

from __future__ import annotations

import dataclasses
from typing import Dict, List

import torch

from ..models.assembled import AssembledModel, CallBinding

_TORCH_DTYPE = {"float32": torch.float32, "bfloat16": torch.bfloat16, "int32": torch.int32}


class CacheStorage:
    def __init__(self, model: AssembledModel, num_pages: int, num_slots: int, page_size: int):
        rt = model.rt
        self.num_pages, self.num_slots, self.page_size = int(num_pages), int(num_slots), int(page_size)
        model.check_page_size(self.page_size)
        self.keys: List[torch.Tensor] = []
        self.values: List[torch.Tensor] = []
        for spec, caches in zip(model.group_specs, model.group_caches):
            for pool, elems in ((self.keys, spec.key_elements(self.page_size)), (self.values, spec.value_elements(self.page_size))):
                # (a mixer may page something else than activations: its cache spec names the pools' dtype then)
                dtype = rt.act_dtype if spec.dtype is None else _TORCH_DTYPE[spec.dtype]
                pool.append(torch.zeros((len(caches), self.num_pages, elems), dtype=dtype, device=rt.device))
        self.states: Dict[int, torch.Tensor] = {}
        for idx, ss in model.state_specs.items():
            self.states[idx] = torch.zeros((self.num_slots, *ss.shape), dtype=_TORCH_DTYPE[ss.dtype], device=rt.device)
        self.bindings: List[CallBinding] = []
        for plan in model.calls:
            call = dataclasses.replace(plan, state=self.states.get(plan.index))
            if call.group >= 0:
                call.k_cache = self.keys[call.group][call.cache_index]
                call.v_cache = self.values[call.group][call.cache_index]
            self.bindings.append(call)

    def nbytes(self) -> int:
        tensors = self.keys + self.values + list(self.states.values())
        return sum(t.numel() * t.element_size() for t in tensors)

    def bytes_per_token(self) -> int:
        """Cache bytes one token occupies over all caches (keys and values)."""
        total = 0
        for t in self.keys + self.values:
            total += t.shape[0] * (t.shape[2] // self.page_size) * t.element_size()
        return total

    def reset_slot(self, slot: int) -> None:
        """Fixed-size state starts from zero when a request takes the slot."""
        for t in self.states.values():
            t[slot].zero_()

    def poison_pages(self, group: int, pages) -> None:
        """Fill the given pages of a group, in all its caches, with NaN (tests: a page that is
        handed out again must be written before it is read)."""
        if len(pages):
            idx = torch.as_tensor(list(pages), dtype=torch.long, device=self.keys[group].device)
            for pool in (self.keys[group], self.values[group]):
                pool[:, idx] = float("nan") if pool.dtype.is_floating_point else -(2 ** 31)
