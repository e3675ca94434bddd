"""A request's state on the host (inference_engine/sequence.py:10-44): its tokens
(prompt, then generated), how many are in the cache, and what it holds there."""
from __future__ import annotations

import enum
import itertools
import time

from ..sampling.params import SamplingParams

_ids = itertools.count()

PENDING = -1     # stands in a request's token list for a token that is being chosen on the device


class Status(enum.Enum):
    WAITING = 0
    RUNNING = 1
    FINISHED = 2


class Sequence:
    def __init__(self, prompt_ids, params: SamplingParams, seed: int | None = None):
        self.seq_id = next(_ids)
        self.token_ids = list(prompt_ids)
        if not self.token_ids:
            raise ValueError("a request needs at least one prompt token")
        self.prompt_len = len(self.token_ids)
        self.params = params
        self.seed = seed if seed is not None else (params.seed if params.seed is not None else self.seq_id)
        self.num_computed = 0            # tokens whose keys and values are in the cache
        self.cache = None                # cache.RequestCache while running
        self.status = Status.WAITING
        self.ending = False              # its last token is on its way (max_tokens or length): schedule no more
        self.num_preemptions = 0
        self.arrival_time = time.perf_counter()
        self.first_token_time: float | None = None
        self.finish_time: float | None = None

    @property
    def num_tokens(self) -> int:
        return len(self.token_ids)

    @property
    def num_new_tokens(self) -> int:
        return self.num_tokens - self.num_computed

    @property
    def output_ids(self) -> list[int]:
        return self.token_ids[self.prompt_len:]

    @property
    def num_output_tokens(self) -> int:
        return self.num_tokens - self.prompt_len

    @property
    def block_table(self) -> list[int]:
        return self.cache.tables[0] if self.cache is not None and self.cache.tables else []
