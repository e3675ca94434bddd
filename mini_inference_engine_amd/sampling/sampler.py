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

import numpy as np
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
    def __init__(self, ops, device, max_rows: int, out: torch.Tensor | None = None):
        """``out``: int32 device buffer of at least ``max_rows`` entries the chosen tokens are written
        to (a fixed address a later step can read them from); by default one is made here."""
        self.ops = ops
        self.device = torch.device(device)
        pin = self.device.type == "cuda"
        # one staging buffer: temperatures (float32 bits), counters, seeds (2 x int32 each)
        self.host = torch.zeros(4 * max_rows, dtype=torch.int32, pin_memory=pin)
        self.host_np = self.host.numpy()
        self.dev = torch.zeros(4 * max_rows, dtype=torch.int32, device=self.device) if pin else self.host
        self.max_rows = max_rows
        self.out = out if out is not None else torch.zeros(max(1, max_rows), dtype=torch.int32, device=self.device)
        # the chosen tokens travel to one of two pinned buffers in turn: the host may still be reading the
        # last step's while this step's copy is queued
        self._landing = [torch.zeros(max(1, max_rows), dtype=torch.int32, pin_memory=pin) for _ in range(2)]
        self._turn = 0
        self._params_copied = None

    def sample_async(self, logits: torch.Tensor, temperatures, seeds, counters) -> ChosenTokens:
        """logits [R, V] float32; python lists of length R.  The tokens are written to ``self.out[:R]``
        and copied towards the host; nothing is waited for."""
        R = logits.shape[0]
        if R > self.max_rows:
            raise ValueError(f"{R} rows to sample, room for {self.max_rows}")
        if self._params_copied is not None:
            self._params_copied.synchronize()        # the staging buffer is free again
        h = self.host_np
        h[:R] = np.asarray(temperatures, dtype=np.float32).view(np.int32)
        h[R:2 * R] = np.asarray(counters, dtype=np.int32)
        h[2 * R:4 * R] = np.asarray([s & 0xFFFFFFFFFFFFFFFF for s in seeds], dtype=np.uint64).view(np.int32)
        if self.dev is not self.host:
            self.dev[:4 * R].copy_(self.host[:4 * R], non_blocking=True)
            self._params_copied = torch.cuda.Event()
            self._params_copied.record()
        temps = self.dev[:R].view(torch.float32)
        ctr = self.dev[R:2 * R]
        sd = self.dev[2 * R:4 * R].view(torch.int64)
        self.ops.sample(logits, temps, sd, ctr, out=self.out[:R])
        if self.dev is self.host:               # no device: everything has happened already; keep a copy, since
            return ChosenTokens(self.out[:R].clone(), None, R, None)     # the next step writes to ``out`` again
        landing = self._landing[self._turn]
        self._turn ^= 1
        landing[:R].copy_(self.out[:R], non_blocking=True)
        ready = torch.cuda.Event()
        ready.record()
        return ChosenTokens(self.out, landing, R, ready)

    def sample(self, logits: torch.Tensor, temperatures, seeds, counters) -> list[int]:
        """The same, waited for: token ids on the host."""
        if logits.shape[0] == 0:
            return []
        return self.sample_async(logits, temperatures, seeds, counters).tolist()
