"""Engine-side knobs (not model constants).

Names and meanings follow the reference's EngineConfig
(inference_engine/config.py:45-56): block_size, max_num_seqs,
max_num_batched_tokens, kv_cache_memory_fraction, max_model_len,
enable_chunked_prefill.  Its Triton and CUDA-graph switches become one
``use_hip_graphs`` switch with ``graph_batch_sizes``; ``num_blocks`` (an explicit
page count), ``num_state_slots``, ``seed`` and ``cast_float32_weights`` have no
counterpart there.
"""
from __future__ import annotations

from dataclasses import dataclass, fields


@dataclass
class EngineConfig:
    block_size: int = 16                    # tokens per cache page
    max_num_seqs: int = 256                 # most requests running at once
    max_num_batched_tokens: int = 2048      # token budget of one step
    kv_cache_memory_fraction: float = 0.85  # of the memory free after the weights
    max_model_len: int = 2048
    enable_chunked_prefill: bool = True
    num_blocks: int | None = None           # explicit page count (scratch page included)
    num_state_slots: int | None = None      # default: max_num_seqs + 1 (slot 0 is scratch)
    use_hip_graphs: bool = True
    # up to 16 rows a step's time grows with every row (13 us a row at TinyLlama sizes), from 17 to 32 hardly: hence 6 and 12
    graph_batch_sizes: tuple = (1, 2, 4, 6, 8, 12, 16, 24, 32, 48, 64, 96, 128, 160, 192, 224, 256)
    portion_graph_sizes: tuple | None = None   # token counts of the captured single-prompt steps; None: eighths of the token budget
    seed: int = 0                           # base of every request's sampling stream
    activation_reserve_bytes: int = 768 * 2**20
    poison_freed_pages: bool = False        # debugging: fill returned pages with NaN
    run_ahead: bool = True                  # start a step before the host has read the tokens of the one before
    tune_library_products: bool = True      # time the library's kernels once for the row counts that recur (graph batch
                                            # sizes, the token budget) and keep the fastest; a few seconds at start-up
    trace_ranges: bool = False              # mark schedule / prepare / forward / sample of every step with profiler ranges
    cast_float32_weights: bool = False      # bfloat16 mode: round tensors the checkpoint stores in 32-bit to bfloat16
                                            # (the reference casts every tensor; by default they stay as stored)

    def __post_init__(self):
        if self.block_size < 16 or self.block_size % 16:
            raise ValueError(f"block_size must be a positive multiple of 16, found {self.block_size}")
        if self.max_num_seqs < 1:
            raise ValueError("max_num_seqs must be >= 1")
        if self.max_num_batched_tokens < 1:
            raise ValueError("max_num_batched_tokens must be >= 1")
        if self.num_blocks is not None and self.num_blocks < 2:
            raise ValueError("num_blocks must be >= 2 (page 0 is scratch)")
        if not 0.0 < self.kv_cache_memory_fraction <= 1.0:
            raise ValueError("kv_cache_memory_fraction must be in (0, 1]")

    @classmethod
    def with_overrides(cls, base: "EngineConfig | None" = None, **overrides) -> "EngineConfig":
        known = {f.name for f in fields(cls)}
        unknown = sorted(set(overrides) - known)
        if unknown:
            raise ValueError(f"unknown EngineConfig fields {unknown}; known: {sorted(known)}")
        values = {f.name: getattr(base, f.name) for f in fields(cls)} if base else {}
        values.update(overrides)
        if "graph_batch_sizes" in values:
            values["graph_batch_sizes"] = tuple(values["graph_batch_sizes"])
        if values.get("portion_graph_sizes") is not None:
            values["portion_graph_sizes"] = tuple(values["portion_graph_sizes"])
        return cls(**values)
