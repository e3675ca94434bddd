"""The step function and what it stands on: model, weights, cache, step arena.

``ModelRunner.forward_step(rows)`` is the one way tokens become logits: generation
(LLMEngine.step), trace replay and the benchmarks all call it.  It runs only the
tokens it is given, as one flattened batch, against the cache earlier steps left,
and returns 32-bit logits at the wanted places in the caller's order.  (The
reference's counterpart is LLMEngine._prepare + LlamaModel.forward,
inference_engine/engine.py:133-201, which returns logits for the last token of
finished prompts only.)
"""
from __future__ import annotations

import torch

from ..cache import CacheManager, CacheStorage, GroupSpec
from ..config.registry import architecture_of, load_model_config
from ..models.decoder import Decoder
from ..weights import load_weights
from .batch import StepArena, StepRow, build_step

_DTYPES = {"bfloat16": torch.bfloat16, "bf16": torch.bfloat16, "float32": torch.float32, "fp32": torch.float32,
           torch.bfloat16: torch.bfloat16, torch.float32: torch.float32}


class PhaseRanges:
    """Named ranges around the phases of a step, for a profiler's timeline (rocprofv3 --marker-trace shows them;
    the reference marks the same four phases with NVTX, inference_engine/engine.py:183-210).  Off by default:
    ``ranges(name)`` is then an empty context."""

    def __init__(self, on: bool = False):
        self.on = bool(on)

    def __call__(self, name: str):
        if self.on:
            return torch.cuda.nvtx.range(name)
        import contextlib
        return contextlib.nullcontext()


def parse_dtype(d) -> torch.dtype:
    if d not in _DTYPES:
        raise ValueError(f"dtype {d!r}: choose bfloat16 or float32")
    return _DTYPES[d]


class ModelRunner:
    def __init__(self, model, *, dtype=torch.bfloat16, device="cuda", backend=None, page_size: int = 16,
                 num_pages: int | None = None, memory_fraction: float = 0.85, reserve_bytes: int = 768 * 2**20,
                 max_step_tokens: int = 2048, max_rows: int = 256, max_model_len: int | None = None,
                 num_state_slots: int | None = None, weights=None, cast_float32_weights: bool = False,
                 tune_library_products: bool = False):
        """``model``: a folder with config.json and safetensors, or a ModelConfig together
        with ``weights`` (name -> tensor).  ``backend``: the kernels; by default the HIP
        library, which must load (there is no other product path)."""
        self.dtype = parse_dtype(dtype)
        self.device = torch.device(device)
        if isinstance(model, str):
            self.model_cfg, arch = load_model_config(model)
            source = model
        else:
            self.model_cfg, arch = model, architecture_of(model)
            if weights is None:
                raise ValueError("a configuration needs weights (name -> tensor) beside it")
            source = weights
        self.model = Decoder(arch.build(self.model_cfg))
        if backend is None:
            from ..kernels.hip_backend import HipBackend
            backend = HipBackend(self.dtype, self.device)
        self.ops = backend
        self.tune_library_products = bool(tune_library_products)
        if self.tune_library_products:
            backend.prefer_rows([max_step_tokens])    # a long prompt comes in portions of exactly the step's token budget
        self.model.use_backend(backend)
        self.load_report = load_weights(self.model, source, self.device, self.dtype, cast_float32=cast_float32_weights)
        self.model.prepare(self.device, self.dtype)

        spec = self.model.spec
        limit = spec.max_position or (1 << 30)
        self.max_model_len = min(max_model_len or limit, limit)
        self.page_size = page_size
        self.max_blocks = -(-self.max_model_len // page_size)
        elem = 2 if self.dtype == torch.bfloat16 else 4
        per_page = self.model.bytes_per_page(page_size, elem)
        n_groups = len(per_page)
        if num_pages is None:
            if self.device.type != "cuda":
                raise ValueError("num_pages must be given off the GPU")
            torch.cuda.empty_cache()
            free, _ = torch.cuda.mem_get_info(self.device)
            budget = int((free - reserve_bytes) * memory_fraction)
            num_pages = max(2, budget // max(1, sum(per_page))) if n_groups else 2
        self.num_pages = int(num_pages)
        self.num_state_slots = int(num_state_slots or max_rows + 1)
        self.cache = CacheManager(page_size, [GroupSpec(w, self.num_pages) for w in self.model.page_groups],
                                  self.num_state_slots)
        self.storage = CacheStorage(self.model, page_size, [self.num_pages] * n_groups, self.num_state_slots,
                                    self.device, self.dtype)
        self.model.attach_cache(self.storage)
        if any(not ce.requirement.paged for ce in self.model.cache_entries.values()):
            self.cache.on_open = self.storage.reset_slot
        self.arena = StepArena(max_step_tokens, max_rows, self.max_blocks, n_groups, self.device)
        self.vocab_size = spec.vocab_size
        # The tokens the last step chose, at a fixed address: the next step's rows may take their token
        # from here on the device (StepRow.taken_from) before the host has seen it.
        self.chosen_tokens = torch.zeros(max(1, max_rows), dtype=torch.int32, device=self.device)
        self.graphs = None                  # captured decode steps, once capture_decode_graphs was called
        self.portion_graphs = []            # captured steps of one prompt portion, by token count (capture_portion_graphs)
        self.last_step_captured = False
        self.ranges = PhaseRanges(False)    # the entry point switches them on (EngineConfig.trace_ranges)

    # ------------------------------------------------------------------ steps
    def build(self, rows: list[StepRow], **kw):
        for r in rows:
            if r.start + len(r.tokens) > self.max_model_len:
                raise ValueError(f"a row reaches position {r.start + len(r.tokens)}, beyond max_model_len "
                                 f"{self.max_model_len}")
            if r.taken_from >= self.chosen_tokens.numel():
                raise ValueError(f"a row takes its token from entry {r.taken_from} of {self.chosen_tokens.numel()}")
        with self.ranges("prepare"):
            step = build_step(rows, self.arena, self.page_size, **kw)
        step.earlier_tokens = self.chosen_tokens
        return step

    def capture_decode_graphs(self, batch_sizes, verbose: bool = False, sample: bool = False) -> None:
        """Capture the forward of a step of single-token rows once per batch size; ``forward_step``
        then replays the smallest captured size that holds such a step instead of launching kernel by
        kernel (inference_engine/engine.py:76-120).  ``sample``: the captured step also chooses a token
        from every row's logits (for callers that pass ``sampling`` to ``forward_step``)."""
        from .graphs import DecodeGraphs
        if self.tune_library_products:
            self.ops.prefer_rows(batch_sizes)     # these row counts recur: the warm-up before each capture may choose kernels
        self.graphs = DecodeGraphs(self, batch_sizes, verbose=verbose, sample=sample)

    def capture_portion_graphs(self, sizes=None) -> None:
        """Capture the step that holds one prompt portion, once for each token count in ``sizes`` (default: the
        step's token budget, what a long prompt is cut into); ``forward_step`` replays the smallest that holds
        such a step: a portion of exactly that many tokens, or, if the model allows padding tokens, a shorter one."""
        from .graphs import PortionGraph
        most = min(self.arena.max_tokens, self.max_model_len)
        sizes = sorted({int(t) for t in (sizes or [self.arena.max_tokens])})
        if not sizes or sizes[0] < 2 or sizes[-1] > most:
            raise ValueError(f"captured portions of {sizes} tokens: between 2 and {most} (the step's budget, the "
                             f"longest request)")
        if self.tune_library_products:
            self.ops.prefer_rows(sizes[-1:])          # the budget's own size recurs with every long prompt
        pool = next(iter(self.graphs.graphs.values()))[0].pool() if self.graphs is not None and self.graphs.graphs else None
        self.portion_graphs = []
        for tokens in reversed(sizes):                # the largest first: the others fit into what it reserved
            self.portion_graphs.append(PortionGraph(self, tokens, pool=pool))
            if pool is None:
                pool = self.portion_graphs[0].graph.pool()
        self.portion_graphs.reverse()

    def _portion_graph_for(self, rows):
        for g in self.portion_graphs:
            if g.takes(rows, self.model.padding_safe):
                return g
        return None

    @torch.inference_mode()
    def forward_step(self, rows: list[StepRow], sampling=None) -> torch.Tensor | None:
        """Logits [sum of wants, vocab] float32, ordered by row then by ``want``.
        Pages for the rows' tokens must have been reserved.

        ``sampling``: (temperatures, seeds, counters), one entry for each wanted row of logits: the step also
        chooses a token from each of them on the device (temperature 0: the largest logit; else a draw whose
        noise is a function of seed and counter) and leaves it in ``chosen_tokens[i]``.  The three arrays
        travel with the step's other arrays, and in a captured step the choice is part of the graph."""
        self.last_step_captured = False
        captured = (self.graphs is not None and self.graphs.fits(len(rows)) and all(len(r.tokens) == 1 for r in rows)
                    and (sampling is None or all(len(r.want) == 1 for r in rows)))
        portion = None if captured or not self.portion_graphs else self._portion_graph_for(rows)
        if portion is not None:
            self.last_step_captured = True
            logits, step = portion.run(self, rows, sampling)
        elif captured:
            self.last_step_captured = True
            logits, step = self.graphs.run(self, rows, sampling)
            if sampling is None or self.graphs.sample:
                return logits
        else:
            step = self.build(rows, sampling=sampling)
            with self.ranges("forward"):
                logits = self.model.forward(step)
        if sampling is not None and logits is not None:
            n = logits.shape[0]
            with self.ranges("sample"):
                self.ops.sample(logits, step.sample_temps[:n], step.sample_seeds[:n], step.sample_counters[:n],
                                out=self.chosen_tokens[:n])
        return logits

    def after_step(self, rows: list[StepRow]) -> None:
        """Tell the cache how far each row's request has come (windows release pages)."""
        for r in rows:
            self.cache.advance(r.cache, r.start + len(r.tokens))
