"""The model that runs a DecoderSpec: embedding, layers in run order, final norm, head.

It is the only forward pass in the engine (generation, replay and benchmarks all
go through ``forward``), and it is the same for every architecture: what differs
between architectures is the DecoderSpec their builder returns.
"""
from __future__ import annotations

from ..parts.base import CacheBinding, CacheRequirement, DecoderSpec, ParamSpec, Part


class CacheEntry:
    """Cache need of one run-order entry that owns a cache."""

    def __init__(self, entry: int, requirement):
        self.entry = entry
        self.requirement = requirement
        self.group = None       # page group id, for requirements that keep data in pages


class Decoder:
    def __init__(self, spec: DecoderSpec):
        self.spec = spec
        self.ops = None
        self.device = None
        self.dtype = None
        # cache needs, one per owning run-order entry; groups by window
        self.cache_entries: dict[int, CacheEntry] = {}
        self.page_groups: list = []       # window (None = all keys) of each page group
        group_keys: list = []
        for e, call in enumerate(spec.schedule):
            if call.cache_of is not None:
                continue
            req = spec.layers[call.layer].mixer.cache_requirement()
            if req is None:
                continue
            if not isinstance(req, CacheRequirement):
                raise TypeError(f"cache_requirement() of layer {call.layer} returned {req!r}, not a CacheRequirement")
            ce = CacheEntry(e, req)
            if req.paged:
                key = req.page_group_key()
                if key not in group_keys:
                    group_keys.append(key)
                    self.page_groups.append(req.window)
                ce.group = group_keys.index(key)
            self.cache_entries[e] = ce
        self.bindings: list[CacheBinding] = []
        # whether a step may carry padding tokens (written to the scratch page): not if a mixer keeps state that
        # every token of a row changes
        self.padding_safe = all(ce.requirement.paged for ce in self.cache_entries.values())

    # ------------------------------------------------------------ structure
    def parts(self):
        seen = set()
        roots = [self.spec.embedding, *self.spec.layers, self.spec.final_norm, self.spec.head]
        for r in roots:
            for p in r.walk():
                if id(p) not in seen:
                    seen.add(id(p))
                    yield p

    def param_specs(self) -> list[tuple[Part, ParamSpec]]:
        return [(p, s) for p in self.parts() for s in p.params()]

    def use_backend(self, ops) -> None:
        self.ops = ops
        for p in self.parts():
            p.ops = ops

    def prepare(self, device, dtype) -> None:
        self.device, self.dtype = device, dtype
        for p in self.parts():
            p.prepare(device, dtype)

    def weight_bytes(self) -> int:
        total, seen = 0, set()
        for p, s in self.param_specs():
            t = getattr(p, s.attr, None)
            if t is not None and t.data_ptr() not in seen:
                seen.add(t.data_ptr())
                total += t.numel() * t.element_size()
        return total

    # ---------------------------------------------------------------- cache
    def bytes_per_page(self, page_size: int, element_size: int) -> list[int]:
        """Bytes one page id costs in each page group (all its entries, K and V)."""
        out = [0] * len(self.page_groups)
        for ce in self.cache_entries.values():
            if ce.group is not None:
                out[ce.group] += ce.requirement.bytes_per_page(page_size, element_size)
        return out

    def attach_cache(self, storage) -> None:
        """``storage`` gives the tensors of each owning entry; readers share them."""
        self.bindings = []
        for e, call in enumerate(self.spec.schedule):
            owner = e if call.cache_of is None else call.cache_of
            ce = self.cache_entries.get(owner)
            if ce is None:
                self.bindings.append(CacheBinding())
                continue
            b = storage.binding(owner)
            self.bindings.append(CacheBinding(group=b.group, k=b.k, v=b.v, state=b.state,
                                              read_only=call.cache_of is not None, page_size=b.page_size,
                                              tensors=b.tensors))

    # -------------------------------------------------------------- forward
    def forward(self, step):
        """Runs exactly the tokens of ``step`` and returns logits [wanted, vocab] in
        32-bit for ``step.logit_rows`` (flat token positions)."""
        spec = self.spec
        residual = spec.embedding.forward(step.input_ids, step.taken_from, step.earlier_tokens)
        h = None
        last = len(spec.schedule) - 1
        for e, (call, binding) in enumerate(zip(spec.schedule, self.bindings)):
            after = spec.final_norm if e == last else spec.layers[spec.schedule[e + 1].layer].first_norm
            h, residual = spec.layers[call.layer].forward(h, residual, step, binding, next_norm=after)
        if step.num_logits == 0:
            return None
        return spec.head.forward(spec.final_norm.lazy(h, residual, rows=step.logit_rows))
