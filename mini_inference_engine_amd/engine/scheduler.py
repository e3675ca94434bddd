"""Which requests run in the next step, and with how many tokens each.

A step is planned against two resources: the token budget of the step and what the cache manager can still
hand out (pages per group, state slots).  The plan is built in three stages, in the order that fixes who
wins when a resource runs short (the behaviour of inference_engine/scheduler.py:57-102):

 1. requests that are running and need exactly one token (they are decoding) get it;
 2. requests that are running and still have part of their prompt to run get the next portion, as large
    as the budget leaves;
 3. waiting requests are admitted first come first served, each with as much of its prompt as the budget
    leaves, unless the step had to evict somebody: then it admits nobody.

Rules of this engine beside those stages:
  * a request whose last token is already on its way (``Sequence.ending``) asks for nothing more;
  * admission takes a state slot as well as pages, and keeps a small share of the pages free for the
    requests already running (not when nothing runs: a request alone may use the last page);
  * when a running request cannot get a page, the request admitted last gives back everything it holds and
    goes to the front of the queue, to be run again from its tokens (inference_engine/scheduler.py:38-55);
    it also leaves the plan of the step if it was in it;
  * what can never run (longer than the cache holds for one request, or stuck at the head of the queue with
    nothing running) raises ``RequestTooLarge`` instead of planning empty steps for ever.
"""
from __future__ import annotations

from collections import deque
from dataclasses import dataclass, field

from ..cache import CacheManager
from ..config.engine_config import EngineConfig
from .sequence import Sequence, Status


class RequestTooLarge(RuntimeError):
    pass


@dataclass
class _Plan:
    """A step being planned: the tokens still to give away and who got how many so far."""
    budget: int
    single: list = field(default_factory=list)       # (request, 1): one row each, first in the step
    portions: list = field(default_factory=list)     # (request, n > 1, or the one token of a prompt of one)
    evicted: bool = False

    def give(self, seq: Sequence, n: int, portion: bool) -> None:
        (self.portions if portion else self.single).append((seq, n))
        self.budget -= n

    def drop(self, seq: Sequence) -> None:
        """``seq`` was evicted after it had been given tokens: they go back to the budget."""
        for rows in (self.single, self.portions):
            for entry in [e for e in rows if e[0] is seq]:
                rows.remove(entry)
                self.budget += entry[1]

    def rows(self) -> list:
        return self.single + self.portions


class Scheduler:
    def __init__(self, cfg: EngineConfig, cache: CacheManager):
        self.cfg = cfg
        self.cache = cache
        self.waiting: deque[Sequence] = deque()
        self.running: list[Sequence] = []            # in order of admission: the last is the first to be evicted
        self.num_preemptions = 0
        # the share of the pages admission leaves to the running requests: about one in a hundred
        groups = range(len(cache.groups))
        self.watermark = max(1, min(cache.usable_pages(g) for g in groups) // 100) if cache.groups else 0

    # ------------------------------------------------------------------ queue
    def add(self, seq: Sequence) -> None:
        room = self.cache.max_tokens_one_request()
        longest = min(seq.prompt_len + seq.params.max_tokens, self.cfg.max_model_len)
        if max(seq.prompt_len, longest) > room:
            raise RequestTooLarge(
                f"request of {seq.prompt_len} prompt + {seq.params.max_tokens} new tokens can never fit: "
                f"the cache holds {room} tokens for one request")
        self.waiting.append(seq)

    def has_work(self) -> bool:
        return bool(self.waiting or self.running)

    # ------------------------------------------------------------------- rules
    def _portion(self, seq: Sequence, budget: int) -> int:
        """Tokens of ``seq`` that may run under ``budget``; 0: not in this step."""
        want = seq.num_new_tokens
        if seq.ending or want <= 0 or budget <= 0:
            return 0
        if want <= budget:
            return want
        return budget if self.cfg.enable_chunked_prefill else 0

    def _evict(self, plan: _Plan) -> Sequence:
        """The request admitted last gives everything back and will be run again from its tokens."""
        victim = self.running.pop()
        self.cache.close(victim.cache)
        victim.cache = None
        victim.num_computed = 0
        victim.status = Status.WAITING
        victim.num_preemptions += 1
        self.num_preemptions += 1
        self.waiting.appendleft(victim)
        plan.drop(victim)
        plan.evicted = True
        return victim

    def _grant(self, seq: Sequence, n: int, plan: _Plan, portion: bool) -> None:
        """Pages for ``n`` more tokens of a running request, evicting from the end of the line until they are
        there; if the line ends at ``seq`` itself it goes too, and gets nothing."""
        while not self.cache.reserve(seq.cache, seq.num_computed, n):
            if self.running[-1] is seq and len(self.running) == 1:
                raise RequestTooLarge(f"request {seq.seq_id} alone cannot get pages for {seq.num_computed + n} tokens")
            if self._evict(plan) is seq:
                return
        plan.give(seq, n, portion)

    def _admit(self, seq: Sequence, n: int, plan: _Plan) -> bool:
        """A state slot and the pages of its first ``n`` tokens, or nothing."""
        if not self.cache.can_open():
            return False
        held = self.cache.open(seq.seq_id)
        keep_free = self.watermark if self.running else 0
        if not self.cache.reserve(held, 0, n, watermark=keep_free):
            self.cache.close(held)
            return False
        seq.cache = held
        seq.status = Status.RUNNING
        self.running.append(seq)
        plan.give(seq, n, portion=True)
        return True

    # ---------------------------------------------------------------- one step
    def schedule(self) -> list[tuple[Sequence, int]]:
        plan = _Plan(self.cfg.max_num_batched_tokens)
        # stages 1 and 2 walk the line as it stood when the step began; who is evicted on the way is skipped
        line = list(self.running)
        for decoding in (True, False):
            for seq in line:
                if seq.status is not Status.RUNNING or (seq.num_new_tokens == 1) != decoding:
                    continue
                n = self._portion(seq, plan.budget)
                if n:
                    self._grant(seq, n, plan, portion=not decoding)
        # stage 3
        while self.waiting and not plan.evicted and len(self.running) < self.cfg.max_num_seqs:
            head = self.waiting[0]
            n = self._portion(head, plan.budget)
            if not n or not self._admit(head, n, plan):
                break
            self.waiting.popleft()

        rows = plan.rows()
        if not rows and self.has_work() and not any(s.ending for s in self.running):
            # (a request whose last token is on its way will make room when it ends)
            raise RequestTooLarge("nothing can be scheduled although requests are waiting: "
                                  "the head of the queue does not fit the cache or the budget")
        return rows

    # ------------------------------------------------------------- after a step
    def advance(self, seq: Sequence, n: int) -> None:
        """``n`` more tokens of ``seq`` are in the cache."""
        seq.num_computed += n
        self.cache.advance(seq.cache, seq.num_computed)

    def finish(self, seq: Sequence) -> None:
        seq.status = Status.FINISHED
        self.running.remove(seq)
        self.cache.close(seq.cache)
        seq.cache = None
