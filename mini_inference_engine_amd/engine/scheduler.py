"""Continuous batching under a token budget, with recompute preemption.

Every step, in this order (inference_engine/scheduler.py:57-102):
 1. each running request with exactly one token to compute gets it;
 2. running requests part-way through their prompt get the next portion, as large
    as the budget allows;
 3. waiting requests are admitted first come first served, each with as much of
    its prompt as the budget still allows, unless something was preempted in this
    very step.
When a running request cannot get a page, the most recently admitted request is
preempted: everything it holds goes back, it returns to the front of the queue
and is later recomputed from its tokens, generated ones included
(inference_engine/scheduler.py:38-55).  Decided beyond the reference: a request
that could never fit raises instead of spinning; requests also hold a state slot,
taken at admission and returned with the pages.
"""
from __future__ import annotations

from collections import deque

from ..cache import CacheManager
from ..config.engine_config import EngineConfig
from .sequence import Sequence, Status


class RequestTooLarge(RuntimeError):
    pass


class Scheduler:
    def __init__(self, cfg: EngineConfig, cache: CacheManager):
        self.cfg = cfg
        self.cache = cache
        self.waiting: deque[Sequence] = deque()
        self.running: list[Sequence] = []
        self.num_preemptions = 0
        # keep about 1% of the pages free at admission so running requests can grow
        self.watermark = max(1, min(cache.usable_pages(g) for g in range(len(cache.groups))) // 100) \
            if cache.groups else 0

    def add(self, seq: Sequence) -> None:
        limit = self.cache.max_tokens_one_request()
        worst = min(seq.prompt_len + seq.params.max_tokens, self.cfg.max_model_len)
        if seq.prompt_len > limit or worst > limit:
            raise RequestTooLarge(
                f"request of {seq.prompt_len} prompt + {seq.params.max_tokens} new tokens can never fit: "
                f"the cache holds {limit} tokens for one request")
        self.waiting.append(seq)

    def has_work(self) -> bool:
        return bool(self.waiting or self.running)

    # ------------------------------------------------------------ preemption
    def _preempt(self, seq: Sequence) -> None:
        self.running.remove(seq)
        self.cache.close(seq.cache)
        seq.cache = None
        seq.num_computed = 0
        seq.status = Status.WAITING
        seq.num_preemptions += 1
        self.num_preemptions += 1
        self.waiting.appendleft(seq)

    def _reserve_or_preempt(self, seq: Sequence, n: int) -> bool:
        """False if ``seq`` itself had to go."""
        while not self.cache.reserve(seq.cache, seq.num_computed, n):
            victim = self.running[-1]
            if victim is seq and len(self.running) == 1:
                raise RequestTooLarge(
                    f"request {seq.seq_id} alone cannot get pages for {seq.num_computed + n} tokens")
            self._preempt(victim)
            if victim is seq:
                return False
        return True

    # -------------------------------------------------------------- one step
    def schedule(self) -> list[tuple[Sequence, int]]:
        budget = self.cfg.max_num_batched_tokens
        decodes, prefills = [], []
        preemptions_before = self.num_preemptions

        for seq in list(self.running):
            if seq.status is not Status.RUNNING or seq.num_new_tokens != 1 or seq.ending:
                continue
            if budget == 0:
                break
            if self._reserve_or_preempt(seq, 1):
                decodes.append((seq, 1))
                budget -= 1

        for seq in list(self.running):
            if seq.status is not Status.RUNNING or seq.num_new_tokens <= 1 or budget == 0 or seq.ending:
                continue
            n = min(seq.num_new_tokens, budget)
            if not self.cfg.enable_chunked_prefill and n < seq.num_new_tokens:
                continue
            if self._reserve_or_preempt(seq, n):
                prefills.append((seq, n))
                budget -= n

        # a request scheduled above may have been preempted to make room afterwards
        decodes = [(s, n) for s, n in decodes if s.status is Status.RUNNING]
        prefills = [(s, n) for s, n in prefills if s.status is Status.RUNNING]

        preempted_now = self.num_preemptions != preemptions_before
        while (self.waiting and budget > 0 and len(self.running) < self.cfg.max_num_seqs and not preempted_now
               and self.cache.can_open()):
            seq = self.waiting[0]
            n = min(seq.num_new_tokens, budget)
            if not self.cfg.enable_chunked_prefill and n < seq.num_new_tokens:
                break
            rc = self.cache.open(seq.seq_id)
            # alone, a request may use the last pages: nothing else is there to grow
            mark = self.watermark if self.running else 0
            if not self.cache.reserve(rc, 0, n, watermark=mark):
                self.cache.close(rc)
                break
            seq.cache = rc
            self.waiting.popleft()
            seq.status = Status.RUNNING
            self.running.append(seq)
            prefills.append((seq, n))
            budget -= n

        if not decodes and not prefills and self.has_work() and not any(s.ending for s in self.running):
            # (a request whose last token is on its way will make room when it ends)
            raise RequestTooLarge("nothing can be scheduled although requests are waiting: "
                                  "the head of the queue does not fit the cache or the budget")
        return decodes + prefills

    def advance(self, seq: Sequence, n: int) -> None:
        """``n`` more tokens of ``seq`` are in the cache."""
        seq.num_computed += n
        self.cache.advance(seq.cache, seq.num_computed)

    def finish(self, seq: Sequence) -> None:
        seq.status = Status.FINISHED
        self.running.remove(seq)
        self.cache.close(seq.cache)
        seq.cache = None
