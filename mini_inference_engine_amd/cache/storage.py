"""Device tensors behind the cache manager's ids.

One K and one V tensor per cache-owning layer call.  Keys: [pages, kv_heads, page, head_dim],
so the keys of one kv head within a page are one contiguous run.  Values:
[pages, kv_heads, head_dim, page], a page's values transposed, so that for one dim the
page's keys are contiguous: both are then what the attention kernels' matrix
instructions take straight from memory.  (The reference keeps
[L, 2, pages, page, kv_heads, head_dim], inference_engine/model.py:43.)  State
entries are [slots, *shape].
"""
from __future__ import annotations

from dataclasses import dataclass

import torch

from ..parts.base import FixedState, PagedKV


@dataclass
class EntryTensors:
    group: int | None
    k: torch.Tensor | None
    v: torch.Tensor | None
    state: torch.Tensor | None
    page_size: int


class CacheStorage:
    def __init__(self, model, page_size: int, pages_per_group: list[int], num_state_slots: int,
                 device, dtype: torch.dtype):
        self.page_size = page_size
        self.entries: dict[int, EntryTensors] = {}
        for e, ce in model.cache_entries.items():
            r = ce.requirement
            if isinstance(r, PagedKV):
                k_shape = (pages_per_group[ce.group], r.num_kv_heads, page_size, r.head_dim)
                v_shape = (pages_per_group[ce.group], r.num_kv_heads, r.head_dim, page_size)
                self.entries[e] = EntryTensors(ce.group, torch.zeros(k_shape, dtype=dtype, device=device),
                                               torch.zeros(v_shape, dtype=dtype, device=device), None, page_size)
            elif isinstance(r, FixedState):
                sd = torch.float32 if r.dtype == "float32" else dtype
                self.entries[e] = EntryTensors(None, None, None, torch.zeros((num_state_slots, *r.shape), dtype=sd,
                                                                            device=device), page_size)

    def binding(self, entry: int) -> EntryTensors:
        return self.entries[entry]

    def poison_pages(self, group: int, pages) -> None:
        """Debugging aid: fill given pages of a group with NaN so a stale read shows."""
        if not pages:
            return
        idx = torch.tensor(list(pages), dtype=torch.long, device=next(iter(self.entries.values())).k.device)
        for t in self.entries.values():
            if t.group == group:
                t.k.index_fill_(0, idx, float("nan"))
                t.v.index_fill_(0, idx, float("nan"))

    def num_bytes(self) -> int:
        n = 0
        for t in self.entries.values():
            for x in (t.k, t.v, t.state):
                if x is not None:
                    n += x.numel() * x.element_size()
        return n
