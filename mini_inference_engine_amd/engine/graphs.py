"""Captured steps: one hipGraph per batch-size bucket of single-token rows, and one per size for a step that
holds a single prompt portion.

A step of single-token rows is launch-bound when run kernel by kernel.  As in the
reference (inference_engine/engine.py:76-120), the whole forward of such a step is
captured once per bucket on static buffers (the step arena) and replayed; a batch is
padded to its bucket with scratch rows that read and write page 0.  Everything a
kernel needs that changes from step to step (token ids, positions, block tables,
slots) is read from the arena on the device, so a replay needs only the arena's
upload.  No memset node is recorded: buffers are cleared by kernels.

A long prompt comes in portions of exactly the token budget of a step; such a step (one row, that many tokens,
starting anywhere in its request, at most one position whose logits are wanted) has the same launches every time
and is captured too (PortionGraph): launched kernel by kernel it costs the host about 3 ms, of which half a
millisecond is not hidden behind the device when the engine was idle.  A shorter prompt, or the rest of a long
one, runs in the smallest captured size that holds it (the entry point captures eighths of the budget), lengthened
with padding tokens: token 0 at the positions that follow, written to the scratch page, which no token of the
prompt itself looks at since they come later; a 512-token prompt then takes what its kernels take instead of what
its launches take.  Not for a model with a mixer whose state every token of a row changes.  The reference captures
single-token steps only.
"""
from __future__ import annotations

import gc
import time

import torch


class DecodeGraphs:
    def __init__(self, runner, batch_sizes, verbose: bool = True, sample: bool = False):
        # The runner owns this object, so it is not kept here: a reference back would make a cycle, and the
        # graphs with all they hold would then be freed whenever the collector runs, possibly in the middle
        # of a later capture, which the runtime does not survive.  ``run`` takes the runner instead.
        arena = runner.arena
        self.sizes = sorted(b for b in set(batch_sizes) if 0 < b <= arena.max_rows and b <= arena.max_tokens)
        self.graphs = {}
        self.static_context = runner.max_model_len
        self.sample = sample               # the captured step also chooses a token from every row's logits
        if not self.sizes:
            return
        t0 = time.perf_counter()
        pool = None
        for bs in reversed(self.sizes):                 # largest first: smaller ones reuse its pool
            step = runner.build([], pad_rows_to=bs, static_context=self.static_context, want_all=True,
                                sampling=([], [], []) if sample else None)
            self._forward(runner, step, bs)             # loads libraries, warms the allocator
            torch.cuda.synchronize()
            g = torch.cuda.CUDAGraph()
            # no garbage collection while the stream records: a collected object that owns device memory
            # or another graph would free it in the middle of the capture
            collecting = gc.isenabled()
            gc.disable()
            try:
                with torch.cuda.graph(g, pool=pool):
                    logits = self._forward(runner, step, bs)
            finally:
                if collecting:
                    gc.enable()
            pool = g.pool()
            self.graphs[bs] = (g, logits)
        torch.cuda.synchronize()
        if verbose:
            print(f"[mini_inference_engine_amd] captured {len(self.sizes)} decode graphs "
                  f"(batch <= {self.sizes[-1]}) in {time.perf_counter() - t0:.1f} s", flush=True)

    def _forward(self, runner, step, bs):
        logits = runner.model.forward(step)
        if self.sample:
            runner.ops.sample(logits, step.sample_temps, step.sample_seeds, step.sample_counters,
                              out=runner.chosen_tokens[:bs])
        return logits

    def fits(self, rows: int) -> bool:
        return bool(self.sizes) and rows <= self.sizes[-1]

    def run(self, runner, rows, sampling=None):
        """``rows``: single-token StepRows.  Logits of the rows that want them, in order, and the step as
        built.  ``sampling`` (one entry a row): with graphs that sample, row i's token is in
        ``runner.chosen_tokens[i]`` afterwards."""
        bs = next(s for s in self.sizes if s >= len(rows))
        picked = [i for i, r in enumerate(rows) if len(r.want)]
        if sampling is None and self.sample:
            sampling = ([0.0] * len(rows), [0] * len(rows), [0] * len(rows))     # nobody reads what is chosen
        step = runner.build(rows, pad_rows_to=bs, static_context=self.static_context, want_all=True, sampling=sampling)
        g, logits = self.graphs[bs]
        with runner.ranges("forward"):       # (and "sample", when the graph chooses the tokens too)
            g.replay()
        if not picked:
            return None, step
        if len(picked) == len(rows):
            return logits[:len(rows)], step
        return logits[torch.tensor(picked, device=logits.device)], step


class _ScratchRequest:
    """What a row needs of a request's cache, all of it the scratch page and the scratch slot: the row a step is
    captured with."""

    def __init__(self, num_groups: int, blocks: int):
        self.tables = [[0] * blocks for _ in range(num_groups)]
        self.state_slot = 0


class PortionGraph:
    """The captured step of one row of ``tokens`` tokens with one row of logits.  It runs a prompt portion of
    exactly that many tokens, or, where the model allows padding tokens (``Decoder.padding_safe``), a shorter
    one lengthened to it."""

    def __init__(self, runner, tokens: int, pool=None):
        from .batch import StepRow
        self.tokens = int(tokens)
        self.static_context = runner.max_model_len
        blocks = -(-self.tokens // runner.page_size)
        scratch = _ScratchRequest(runner.arena.num_groups, blocks)
        row = StepRow(scratch, [0] * self.tokens, 0, [self.tokens - 1])
        step = runner.build([row], static_context=self.static_context)
        runner.model.forward(step)                      # loads libraries, chooses the library's kernels, warms the allocator
        torch.cuda.synchronize()
        self.graph = torch.cuda.CUDAGraph()
        collecting = gc.isenabled()
        gc.disable()                                    # (as for the decode graphs: nothing is collected while the stream records)
        try:
            with torch.cuda.graph(self.graph, pool=pool):
                self.logits = runner.model.forward(step)
        finally:
            if collecting:
                gc.enable()
        torch.cuda.synchronize()

    def takes(self, rows, padding_safe: bool = False) -> bool:
        if len(rows) != 1 or len(rows[0].want) > 1 or rows[0].taken_from >= 0:
            return False
        n = len(rows[0].tokens)
        return n == self.tokens or (padding_safe and 2 <= n < self.tokens
                                    and rows[0].start + self.tokens <= self.static_context)

    def run(self, runner, rows, sampling=None):
        """Logits [1, vocab] of the row's wanted position (None if it wants none), and the step as built."""
        from .batch import StepRow
        row = rows[0]
        wanted = bool(len(row.want))
        if not wanted:                                  # the graph computes one row of logits whatever happens: the last token's
            row = StepRow(row.cache, row.tokens, row.start, [len(row.tokens) - 1])
        step = runner.build([row], static_context=self.static_context, sampling=sampling if wanted else None,
                            pad_portion_to=self.tokens)
        with runner.ranges("forward"):
            self.graph.replay()
        return (self.logits if wanted else None), step
