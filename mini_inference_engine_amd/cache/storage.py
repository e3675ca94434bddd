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


@dataclass
class EntryTensors:
    group: int | None
    k: torch.Tensor | None
    v: torch.Tensor | None
    state: torch.Tensor | None
    page_size: int
    tensors: dict | None = None        # everything the requirement allocated, by name
    requirement: object = None


class CacheStorage:
    def __init__(self, model, page_size: int, pages_per_group: list[int], num_state_slots: int,
                 device, dtype: torch.dtype):
        """Every cache-owning layer call's requirement allocates its own tensors (parts.base.CacheRequirement);
        this class only keeps them and knows which belong to which page group."""
        self.page_size = page_size
        self.device = torch.device(device)
        self.entries: dict[int, EntryTensors] = {}
        for e, ce in model.cache_entries.items():
            r = ce.requirement
            pages = pages_per_group[ce.group] if ce.group is not None else 0
            t = r.allocate(pages, page_size, num_state_slots, device, dtype)
            self.entries[e] = EntryTensors(ce.group, t.get("k"), t.get("v"), t.get("state"), page_size, t, r)

    def binding(self, entry: int) -> EntryTensors:
        return self.entries[entry]

    def reset_slot(self, slot: int) -> None:
        """A state slot is handed to a request: every entry with state of fixed size starts it afresh."""
        for t in self.entries.values():
            t.requirement.reset_slot(t.tensors, slot)

    def poison_pages(self, group: int, pages) -> None:
        """Debugging aid: fill given pages of a group with NaN so a stale read shows."""
        if not pages:
            return
        idx = torch.tensor(list(pages), dtype=torch.long, device=self.device)
        for t in self.entries.values():
            if t.group == group:
                for x in t.tensors.values():
                    if x.is_floating_point():
                        x.index_fill_(0, idx, float("nan"))

    def num_bytes(self) -> int:
        return sum(x.numel() * x.element_size() for t in self.entries.values() for x in t.tensors.values())
