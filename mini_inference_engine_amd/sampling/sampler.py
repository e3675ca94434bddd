"""Choosing the next token of every row that finished its known tokens.

The reference takes argmax, or argmax(softmax(logits / t) / E) with E ~ Exp(1)
drawn by the device generator (inference_engine/sampling.py:13-22); taking logs,
that race is argmax(logits / t + g) with Gumbel noise g.  Here g comes from a
counter-based hash of (request seed, index of the output token, vocabulary
index), so a request's draws do not depend on what else is in the batch, on how
its prompt was cut, or on a preemption in between, and one kernel serves greedy
and sampled rows alike with no host-side branch on the temperatures.
"""
from __future__ import annotations

import torch


class ChosenTokens:
    """Tokens a step chose, on their way to the host."""

    def __init__(self, device_tokens, host_tokens, count, ready):
        self.device_tokens, self._host, self._count, self._ready = device_tokens, host_tokens, count, ready

    def tolist(self) -> list[int]:
        """Waits for the copy (the one device -> host wait of a step)."""
        if self._ready is not None:
            self._ready.synchronize()
            return self._host[:self._count].tolist()
        return self.device_tokens[:self._count].tolist()


class Sampler:
    """Brings the tokens a step chose to the host.  The choice itself happens in the step (the runner's
    ``forward_step(rows, sampling=...)``: its inputs travel with the step's other arrays, and a captured step
    chooses inside its graph); ``sampling_inputs`` makes those inputs from the requests."""

    def __init__(self, device, max_rows: int, out: torch.Tensor):
        """``out``: the int32 device buffer the chosen tokens are written to (a fixed address a later step
        can read them from)."""
        self.device = torch.device(device)
        pin = self.device.type == "cuda"
        self.max_rows = max_rows
        self.out = out
        # the chosen tokens travel to one of two pinned buffers in turn: the host may still be reading the
        # last step's while this step's copy is queued
        self._landing = [torch.zeros(max(1, max_rows), dtype=torch.int32, pin_memory=pin) for _ in range(2)]
        self._turn = 0

    @staticmethod
    def sampling_inputs(seqs):
        """(temperatures, seeds, counters) of the requests a token is chosen for: the counter is the index of the
        output token, so a request's draws do not depend on how it was batched, cut or preempted."""
        return ([s.params.temperature for s in seqs], [s.seed for s in seqs], [s.num_output_tokens for s in seqs])

    def fetch_async(self, count: int) -> ChosenTokens:
        """The first ``count`` chosen tokens on their way to the host; nothing is waited for."""
        if count > self.max_rows:
            raise ValueError(f"{count} chosen tokens, room for {self.max_rows}")
        if self.device.type != "cuda":       # no device: everything has happened already; keep a copy, since
            return ChosenTokens(self.out[:count].clone(), None, count, None)     # the next step writes to ``out`` again
        landing = self._landing[self._turn]
        self._turn ^= 1
        landing[:count].copy_(self.out[:count], non_blocking=True)
        ready = torch.cuda.Event()
        ready.record()
        return ChosenTokens(self.out, landing, count, ready)
