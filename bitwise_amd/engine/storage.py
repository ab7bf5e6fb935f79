"""Device memory behind the cache manager: for every cache group one pool of key pages and
one of value pages per cache, and for every layer call with per-request state one tensor
with a row per slot (the role of KVPool, src/model.h:64-76; zero-initialised as
src/model.cpp:246-247).  Page p of a group is the same page number in all of its caches.
"""

from __future__ import annotations

from typing import Dict, List

import torch

from ..models.assembled import AssembledModel

_TORCH_DTYPE = {"float32": torch.float32, "bfloat16": torch.bfloat16, "int32": torch.int32}


class CacheStorage:
    def __init__(self, model: AssembledModel, num_pages: int, num_slots: int):
        rt = model.rt
        self.num_pages, self.num_slots, self.page_size = num_pages, num_slots, rt.page_size
        self.keys: List[torch.Tensor] = []
        self.values: List[torch.Tensor] = []
        for spec, caches in zip(model.group_specs, model.group_caches):
            page_elems = spec.kv_heads * rt.page_size * spec.head_dim
            shape = (len(caches), num_pages, page_elems)
            self.keys.append(torch.zeros(shape, dtype=rt.act_dtype, device=rt.device))
            self.values.append(torch.zeros(shape, dtype=rt.act_dtype, device=rt.device))
        self.states: Dict[int, torch.Tensor] = {}
        for idx, ss in model.state_specs.items():
            self.states[idx] = torch.zeros((num_slots, *ss.shape), dtype=_TORCH_DTYPE[ss.dtype], device=rt.device)
        for call in model.calls:
            if call.group >= 0:
                call.k_cache = self.keys[call.group][call.cache_index]
                call.v_cache = self.values[call.group][call.cache_index]
            call.state = self.states.get(call.index)

    def nbytes(self) -> int:
        tensors = self.keys + self.values + list(self.states.values())
        return sum(t.numel() * t.element_size() for t in tensors)

    def bytes_per_token(self) -> int:
        """Cache bytes one token occupies over all caches (keys and values)."""
        total = 0
        for k in self.keys:
            total += 2 * k.shape[0] * (k.shape[2] // self.page_size) * k.element_size()
        return total

    def reset_slot(self, slot: int) -> None:
        """Fixed-size state starts from zero when a request takes the slot."""
        for t in self.states.values():
            t[slot].zero_()
