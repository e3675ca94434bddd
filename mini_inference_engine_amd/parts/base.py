"""Interfaces of the parts a decoder is put together from.

A part owns its sizes and constants as constructor parameters, declares the
checkpoint tensors it wants (``params``), says what cache it needs
(``cache_requirement``, mixers only) and computes through a kernel backend
(``self.ops``) that the model hands to every part.  No part knows which model
it is in, which layer it is, or what the other layers are.

Interfaces
----------
Norm.forward(x, residual, rows=None) -> y
    ``residual`` is the fp32 stream [T, width]; ``x`` (or None) is the branch
    output still to be added to it.  Adds in place, normalises, returns ``y`` in
    the activation dtype.  With ``rows`` (int32 indices) only those rows are
    produced and the stream is left untouched.  Norm.lazy(...) returns the same
    as a kernels.api.Normed, for parts that set ``lazy_input`` and hand it to
    their first ``ops.linear`` (norm and product then run as one kernel).
PositionEncoding.encode_and_store(ops, qkv, step, n_q_heads, n_kv_heads, k_cache, v_cache, slots)
    Encodes q and k inside the fused projection output in place, as a function of
    each token's absolute position only, and writes k, v to the cache.
    project_encode_store(ops, x, w_qkv, ...) does the projection too (default: linear,
    then encode_and_store) and returns a tensor whose first Hq * D columns are q.
Mixer.forward(x, step, cache, add_to=None) -> y or None     [T, width] -> [T, width]
    Must accept a portion that starts anywhere in a request and leave its cache
    or state as if the request had been fed whole.  ``add_to`` (a kernels.api.Sink)
    is where the block will add y: a part may pass it to its last ``ops.linear`` and
    return what that returns (None or a Normed = already added), or ignore it and return y.
FeedForward.forward(x, step, add_to=None) -> y or None       token-wise
Block.forward(h, residual, step, cache, next_norm=None) -> (h, residual)
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Sequence


@dataclass(frozen=True)
class Source:
    """One piece of a device buffer and the checkpoint tensor it comes from.

    ``shape`` is the piece as it lands in the buffer, ``row_offset`` where its rows go inside a stacked buffer.
    By default the piece is the whole checkpoint tensor ``name``.  A checkpoint that stores things differently
    is declared, not special-cased in the loader:
      stored_shape   shape of the checkpoint tensor, where it differs from ``shape``
      rows, cols     (start, stop): the part of the stored tensor's dim 0 / dim 1 this piece takes (a fused
                     tensor of the checkpoint split over several buffers; several Sources may name one tensor)
      transform      name of a registered function (register_weight_transform) applied to the slice; its
                     result must have ``shape`` ("transpose" ships: a matrix stored [in, out])
    """
    name: str
    shape: tuple
    row_offset: int = 0
    stored_shape: tuple | None = None
    rows: tuple | None = None
    cols: tuple | None = None
    transform: str | None = None

    @property
    def checkpoint_shape(self) -> tuple:
        return tuple(self.stored_shape) if self.stored_shape is not None else tuple(self.shape)


# name -> function(tensor) -> tensor, applied by the loader to a Source's slice of its checkpoint tensor
WEIGHT_TRANSFORMS: dict = {"transpose": lambda t: t.t()}


def register_weight_transform(name: str, fn) -> None:
    """A way a checkpoint stores a tensor differently from how a part wants it (per-head interleaving, [in, out]
    matrices, ...), by name, so that a part can ask for it in a Source from outside the package too."""
    WEIGHT_TRANSFORMS[name] = fn


@dataclass(frozen=True)
class ParamSpec:
    """A device buffer a part wants filled: one source, or several stacked on dim 0."""
    attr: str
    shape: tuple
    sources: tuple
    integer: bool = False   # integer tables are kept as int32
    init: str = "weight"    # how the random-weights mode draws it: "weight" N(0, std), "scale" 1 + N(0, std), "zeros";
                            # integer tables: uniform in [0, integer_bound)
    integer_bound: int = 0  # random-weights mode: an integer table's entries are drawn below this

    @staticmethod
    def single(attr: str, name: str, shape: Sequence[int], integer: bool = False, init: str = "weight",
               integer_bound: int = 0) -> "ParamSpec":
        shape = tuple(int(s) for s in shape)
        return ParamSpec(attr, shape, (Source(name, shape, 0),), integer, init, integer_bound)

    @staticmethod
    def stacked(attr: str, pieces: Sequence) -> "ParamSpec":
        """pieces, in row order: (name, shape) for a whole checkpoint tensor, or a Source (whose row_offset is
        set here) for a slice or a transformed tensor; all share the trailing dims."""
        sources, off = [], 0
        first = pieces[0]
        tail = tuple((first.shape if isinstance(first, Source) else first[1])[1:])
        for piece in pieces:
            src = piece if isinstance(piece, Source) else Source(piece[0], tuple(int(s) for s in piece[1]))
            shape = tuple(int(s) for s in src.shape)
            if tuple(shape[1:]) != tail:
                raise ValueError(f"cannot stack {src.name} {shape} on tail {tail}")
            sources.append(Source(src.name, shape, off, src.stored_shape, src.rows, src.cols, src.transform))
            off += shape[0]
        return ParamSpec(attr, (off,) + tail, tuple(sources))


class Part:
    """Base of all parts: parameter declaration, children, backend injection."""

    ops: Any = None

    def params(self) -> list[ParamSpec]:
        return []

    def children(self) -> list["Part"]:
        return []

    def walk(self):
        yield self
        for c in self.children():
            yield from c.walk()

    def bind(self, attr: str, tensor) -> None:
        setattr(self, attr, tensor)

    def prepare(self, device, dtype) -> None:
        """Build derived device tables (none by default)."""

    def use_backend(self, ops) -> None:
        for p in self.walk():
            p.ops = ops


# ---------------------------------------------------------------- cache needs
class CacheRequirement:
    """What a mixer call wants kept between steps.  The model, the cache manager and the storage know no
    kind by name: they ask the requirement.  A new kind (another layout per token, a latent instead of
    keys and values, several state tensors) is a subclass; nothing else changes.

    paged        True: data per token, in pages that the cache manager hands out per request; requirements
                 with equal ``page_group_key()`` share page ids and block tables.  What a token writes goes to its
                 slot only, so a step may carry padding tokens that write to the scratch page (a model all of
                 whose requirements are paged can run a prompt portion in a captured step of more tokens).
    window       for paged data: how many keys back a query looks at most (None = all); pages that lie
                 wholly before the window are given back.
    bytes_per_page(page_size, element_size)   what one page id costs in this entry (sizes the pool)
    allocate(num_pages, page_size, num_slots, device, act_dtype) -> dict of tensors, handed to the mixer as
                 CacheBinding.k / .v / .state (keys of those names) and CacheBinding.tensors (all of them)
    reset_slot(tensors, slot)   state of fixed size: called when a slot is handed to a request
    """
    paged = False
    window = None

    def page_group_key(self):
        return self.window

    def bytes_per_page(self, page_size: int, element_size: int) -> int:
        return 0

    def allocate(self, num_pages: int, page_size: int, num_slots: int, device, act_dtype) -> dict:
        raise NotImplementedError

    def reset_slot(self, tensors: dict, slot: int) -> None:
        pass


@dataclass(frozen=True)
class PagedKV(CacheRequirement):
    """Keys and values of every token in pages; ``window`` keys back at most, or all.  Keys
    [pages, kv_heads, page, head_dim]; values [pages, kv_heads, head_dim, page] (a page's values transposed:
    both are then what the attention kernels' matrix instructions take straight from memory)."""
    num_kv_heads: int
    head_dim: int
    window: int | None = None
    paged = True

    def bytes_per_page(self, page_size, element_size):
        return 2 * page_size * self.num_kv_heads * self.head_dim * element_size

    def allocate(self, num_pages, page_size, num_slots, device, act_dtype):
        import torch
        return {"k": torch.zeros((num_pages, self.num_kv_heads, page_size, self.head_dim), dtype=act_dtype, device=device),
                "v": torch.zeros((num_pages, self.num_kv_heads, self.head_dim, page_size), dtype=act_dtype, device=device)}


@dataclass(frozen=True)
class FixedState(CacheRequirement):
    """Per-request state of fixed size, [slots, *shape], indexed by the request's state slot; zeroed when
    the slot is handed to a request.  ``dtype``: 'float32' or 'activation'."""
    shape: tuple
    dtype: str = "float32"

    def allocate(self, num_pages, page_size, num_slots, device, act_dtype):
        import torch
        dt = torch.float32 if self.dtype == "float32" else act_dtype
        return {"state": torch.zeros((num_slots, *self.shape), dtype=dt, device=device)}

    def reset_slot(self, tensors, slot):
        tensors["state"][slot].zero_()


@dataclass
class CacheBinding:
    """What a mixer call gets: the tensors of the cache entry it reads/writes."""
    group: int | None = None          # page group id (PagedKV) or None
    k: Any = None                     # [pages, kv_heads, page, head_dim]
    v: Any = None
    state: Any = None                 # [slots, *shape]
    read_only: bool = False           # entry belongs to another layer call
    page_size: int = 0
    tensors: Any = None               # everything the requirement allocated, by name


class Norm(Part):
    width: int

    def forward(self, x, residual, rows=None):
        raise NotImplementedError

    def lazy(self, x, residual, rows=None):
        """The same result, deferred (kernels.api.Normed)."""
        raise NotImplementedError


class PositionEncoding(Part):
    def encode_and_store(self, ops, qkv, step, num_q_heads, num_kv_heads, k_cache, v_cache, slots):
        raise NotImplementedError

    def project_encode_store(self, ops, x, w_qkv, step, num_q_heads, num_kv_heads, k_cache, v_cache, slots):
        """Default: the projection, then encode_and_store on its output."""
        qkv = ops.linear(x, w_qkv)
        self.encode_and_store(ops, qkv, step, num_q_heads, num_kv_heads, k_cache, v_cache, slots)
        return qkv


class Mixer(Part):
    lazy_input = False      # True: forward takes a Normed and gives it to its first ops.linear

    def cache_requirement(self):
        return None

    def forward(self, x, step, cache: CacheBinding, add_to=None):
        raise NotImplementedError


class FeedForward(Part):
    lazy_input = False

    def forward(self, x, step, add_to=None):
        raise NotImplementedError


class Block(Part):
    mixer: Mixer
    first_norm = None       # the norm a block applies to the stream first, if it wants the block before it to know

    def forward(self, h, residual, step, cache: CacheBinding, next_norm=None):
        raise NotImplementedError


# ------------------------------------------------------------ part registries
# Kind name -> class, so that a configuration can choose a part layer by layer
# and a new kind can be added from outside the package.
MIXERS: dict[str, type] = {}
FEED_FORWARDS: dict[str, type] = {}
NORMS: dict[str, type] = {}
POSITION_ENCODINGS: dict[str, type] = {}
BLOCKS: dict[str, type] = {}


def _register(table: dict, kind: str):
    def deco(cls):
        table[kind] = cls
        cls.kind = kind
        return cls
    return deco


def register_mixer(kind: str):
    return _register(MIXERS, kind)


def register_feed_forward(kind: str):
    return _register(FEED_FORWARDS, kind)


def register_norm(kind: str):
    return _register(NORMS, kind)


def register_position_encoding(kind: str):
    return _register(POSITION_ENCODINGS, kind)


def register_block(kind: str):
    return _register(BLOCKS, kind)


@dataclass(frozen=True)
class LayerCall:
    """One entry of the run order: which layer runs, and whose cache it uses.
    ``cache_of`` names an earlier entry of the run order whose cache this call
    reads instead of owning one."""
    layer: int
    cache_of: int | None = None


@dataclass
class DecoderSpec:
    """A whole model as data: parts plus the order in which layers run."""
    embedding: Part
    layers: list
    final_norm: Norm
    head: Part
    schedule: list = field(default_factory=list)
    ignore_tensors: tuple = ()      # regular expressions of checkpoint names to skip
    stop_token_ids: tuple = ()      # a request ends when it draws one of these (unless told to ignore them)
    max_position: int | None = None
    vocab_size: int = 0

    def __post_init__(self):
        if not self.schedule:
            self.schedule = [LayerCall(i) for i in range(len(self.layers))]
        owners = set()
        for e, call in enumerate(self.schedule):
            if not 0 <= call.layer < len(self.layers):
                raise ValueError(f"run order entry {e} names layer {call.layer}; there are {len(self.layers)}")
            if call.cache_of is None:
                owners.add(e)
            elif call.cache_of not in owners or call.cache_of >= e:
                raise ValueError(f"run order entry {e} reads the cache of entry {call.cache_of}, "
                                 "which must be an earlier entry that owns one")
