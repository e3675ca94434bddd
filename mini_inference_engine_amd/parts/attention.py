"""Grouped-query softmax attention over a paged cache.

qkv = x W_qkv^T, split [Hq D, Hkv D, Hkv D]; q, k position-encoded; k, v written
to the cache before attention; query head i reads kv head i // (Hq / Hkv); a
query at position p sees keys max(0, p - window + 1) .. p of its own request;
scores * scale, softmax in 32-bit, times V; then the output projection
(inference_engine/model.py:122-159,172-178).  ``window`` None = all keys (the
reference has no window).  With ``has_kv`` False the part projects only q and
must be given another call's cache to read.
"""
from __future__ import annotations

from .base import Mixer, PagedKV, ParamSpec, register_mixer


@register_mixer("attention")
class Attention(Mixer):
    lazy_input = True

    def __init__(self, width: int, num_heads: int, num_kv_heads: int, head_dim: int, scale: float,
                 position, prefix: str, window: int | None = None, has_kv: bool = True):
        if num_heads % num_kv_heads:
            raise ValueError(f"{num_heads} query heads are not a multiple of {num_kv_heads} kv heads")
        if head_dim % 16 or not 16 <= head_dim <= 256:
            raise ValueError(f"head_dim {head_dim}: the attention kernels take multiples of 16 from 16 to 256")
        if window is not None and window < 1:
            raise ValueError("window must be >= 1 or None")
        self.width = int(width)
        self.num_heads = int(num_heads)
        self.num_kv_heads = int(num_kv_heads)
        self.head_dim = int(head_dim)
        self.scale = float(scale)
        self.position = position
        self.prefix = prefix
        self.window = window
        self.has_kv = bool(has_kv)
        self.w_qkv = None
        self.w_o = None

    def children(self):
        return [self.position] if self.position is not None else []

    def params(self):
        p, d, w = self.prefix, self.head_dim, self.width
        pieces = [(f"{p}.q_proj.weight", (self.num_heads * d, w))]
        if self.has_kv:
            pieces += [(f"{p}.k_proj.weight", (self.num_kv_heads * d, w)),
                       (f"{p}.v_proj.weight", (self.num_kv_heads * d, w))]
        return [ParamSpec.stacked("w_qkv", pieces),
                ParamSpec.single("w_o", f"{p}.o_proj.weight", (w, self.num_heads * d))]

    def cache_requirement(self):
        return PagedKV(self.num_kv_heads, self.head_dim, self.window)

    def forward(self, x, step, cache, add_to=None):
        ops = self.ops
        if cache.read_only == self.has_kv:
            raise ValueError("an attention part with k/v projections owns its cache; one without reads another's")
        group = step.groups[cache.group]
        kv_heads_in_row = self.num_kv_heads if self.has_kv else 0
        k_cache, v_cache, slots = (cache.k, cache.v, group.slot_mapping) if self.has_kv else (None, None, None)
        qkv = self.position.project_encode_store(ops, x, self.w_qkv, step, self.num_heads, kv_heads_in_row,
                                                 k_cache, v_cache, slots)
        out = ops.paged_attention(qkv, self.num_heads, self.num_kv_heads, self.head_dim, cache.k, cache.v,
                                  group, step, self.scale, self.window)
        return ops.linear(out, self.w_o, add_to=add_to)
