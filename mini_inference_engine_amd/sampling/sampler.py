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


class Sampler:
    def __init__(self, ops, device, max_rows: int):
        self.ops = ops
        self.device = torch.device(device)
        pin = self.device.type == "cuda"
        # one staging buffer: temperatures (float32 bits), counters, seeds (2 x int32 each)
        self.host = torch.zeros(4 * max_rows, dtype=torch.int32, pin_memory=pin)
        self.host_np = self.host.numpy()
        self.dev = torch.zeros(4 * max_rows, dtype=torch.int32, device=self.device) if pin else self.host
        self.max_rows = max_rows

    def sample(self, logits: torch.Tensor, temperatures, seeds, counters) -> list[int]:
        """logits [R, V] float32; python lists of length R.  Returns token ids (host)."""
        R = logits.shape[0]
        if R == 0:
            return []
        if R > self.max_rows:
            raise ValueError(f"{R} rows to sample, room for {self.max_rows}")
        h = self.host_np
        h[:R] = np.asarray(temperatures, dtype=np.float32).view(np.int32)
        h[R:2 * R] = np.asarray(counters, dtype=np.int32)
        h[2 * R:4 * R] = np.asarray([s & 0xFFFFFFFFFFFFFFFF for s in seeds], dtype=np.uint64).view(np.int32)
        if self.dev is not self.host:
            self.dev[:4 * R].copy_(self.host[:4 * R], non_blocking=True)
        temps = self.dev[:R].view(torch.float32)
        ctr = self.dev[R:2 * R]
        sd = self.dev[2 * R:4 * R].view(torch.int64)
        tokens = self.ops.sample(logits, temps, sd, ctr)
        return tokens.tolist()      # the one device -> host wait of a step
