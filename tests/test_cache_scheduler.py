"""The cache manager and the scheduler's decisions, on the host alone.

Invariants checked under random orders of requests: no page is lost, held twice or
given back twice; the free list plus all tables plus the scratch page make the pool;
windowed groups give pages back as the window passes them; a step never exceeds the
token budget; single tokens come before portions; a preempted request returns to the
front and resumes with the same tokens; a request that can never fit raises.
"""
import random

import pytest

from mini_inference_engine_amd.cache import CacheAccountingError, CacheManager, GroupSpec, IdPool
from mini_inference_engine_amd.config import EngineConfig
from mini_inference_engine_amd.engine.scheduler import RequestTooLarge, Scheduler
from mini_inference_engine_amd.engine.sequence import Sequence, Status
from mini_inference_engine_amd.sampling import SamplingParams


# ------------------------------------------------------------------------ pools
def test_pool_hands_out_lowest_first_and_reuses_in_release_order():
    """inference_engine/block_manager.py:19,39,43 there: page 0 reserved, popleft / extend."""
    pool = IdPool(6)
    assert pool.take(3) == [1, 2, 3]
    pool.give_back([2])
    assert pool.take(3) == [4, 5, 2]
    assert pool.take(1) is None and pool.num_free == 0
    with pytest.raises(CacheAccountingError):
        pool.give_back([0])                      # scratch
    pool.give_back([4])
    with pytest.raises(CacheAccountingError):
        pool.give_back([4])                      # twice
    assert pool.low_water == 0


def manager(pages=20, page=16, windows=(None,), slots=8):
    return CacheManager(page, [GroupSpec(w, pages) for w in windows], slots)


def test_pages_needed_rule():
    """max(0, ceil((computed + n) / page) - len(table)), inference_engine/block_manager.py:25-27 there."""
    cm = manager()
    rc = cm.open("a")
    assert cm.pages_needed(rc, 0, 1) == [1] and cm.pages_needed(rc, 0, 16) == [1] and cm.pages_needed(rc, 0, 17) == [2]
    assert cm.reserve(rc, 0, 17) and len(rc.tables[0]) == 2
    assert cm.pages_needed(rc, 17, 15) == [0] and cm.pages_needed(rc, 17, 16) == [1]
    assert cm.reserve(rc, 17, 15) and len(rc.tables[0]) == 2
    cm.check()


def test_reservation_is_all_or_nothing_across_groups():
    cm = CacheManager(16, [GroupSpec(None, 10), GroupSpec(32, 4)], 4)
    rc = cm.open("a")
    assert cm.reserve(rc, 0, 48)                       # 3 pages in each group; the windowed pool has 3 usable
    rc2 = cm.open("b")
    assert not cm.reserve(rc2, 0, 16)                  # group 1 is empty: nothing is taken from group 0 either
    assert cm.num_free(0) == 6 and rc2.tables == [[], []]
    cm.check()


def test_watermark_only_counts_when_pages_are_needed():
    cm = manager(pages=5)                              # 4 usable
    rc = cm.open("a")
    assert not cm.reserve(rc, 0, 48, watermark=2)      # 4 - 3 < 2
    assert cm.reserve(rc, 0, 32, watermark=2)
    assert cm.reserve(rc, 32, 0 + 0, watermark=99) and cm.reserve(rc, 16, 16, watermark=99)   # nothing needed


def test_state_slots_follow_the_request():
    cm = manager(slots=3)                              # 2 usable
    a, b = cm.open("a"), cm.open("b")
    assert {a.state_slot, b.state_slot} == {1, 2} and not cm.can_open()
    with pytest.raises(CacheAccountingError):
        cm.open("c")
    cm.close(a)
    assert cm.can_open() and cm.open("c").state_slot == 1
    with pytest.raises(CacheAccountingError):
        cm.close(a)                                    # twice
    with pytest.raises(CacheAccountingError):
        cm.open("b")                                   # already open
    cm.check()


def test_window_gives_pages_back_as_it_passes():
    cm = CacheManager(16, [GroupSpec(None, 40), GroupSpec(20, 40)], 4)
    rc = cm.open("a")
    pos = 0
    for n in (16, 16, 16, 16, 1, 1, 1, 30):
        assert cm.reserve(rc, pos, n)
        pos += n
        cm.advance(rc, pos)
        cm.check()
        full, win = rc.tables
        assert len(full) == len(win) == -(-pos // 16) and 0 not in full
        first_key = max(0, pos - 20 + 1)               # the next query sits at pos and sees keys from here
        for i, p in enumerate(win):
            assert (p == 0) == ((i + 1) * 16 <= first_key), f"page {i} at {pos} tokens"
    held = sum(1 for p in rc.tables[1] if p)
    assert held <= 20 // 16 + 2
    cm.close(rc)
    cm.check()
    assert cm.num_free(0) == 39 and cm.num_free(1) == 39


@pytest.mark.parametrize("seed", range(6))
def test_no_page_lost_or_held_twice_under_random_traffic(seed):
    rng = random.Random(seed)
    cm = CacheManager(16, [GroupSpec(None, 30), GroupSpec(24, 30)], 6)
    live = {}
    for step in range(400):
        action = rng.random()
        if action < 0.25 and cm.can_open():
            rid = f"r{step}"
            live[rid] = [cm.open(rid), 0]
        elif action < 0.85 and live:
            rid = rng.choice(list(live))
            rc, pos = live[rid]
            n = rng.choice([1, 1, 1, 2, 5, 16, 17, 40])
            if cm.reserve(rc, pos, n):
                live[rid][1] = pos + n
                cm.advance(rc, pos + n)
            else:
                before = [list(t) for t in rc.tables]
                assert rc.tables == before, "a failed reservation must take nothing"
        elif live:
            rid = rng.choice(list(live))
            cm.close(live.pop(rid)[0])
        cm.check()
    for rc, _ in live.values():
        cm.close(rc)
    cm.check()
    assert cm.num_free(0) == 29 and cm.num_free(1) == 29 and cm.slots.num_free == 5


# -------------------------------------------------------------------- scheduler
def make(pages=40, budget=2048, seqs=256, chunked=True, page=16, max_len=2048):
    cfg = EngineConfig(block_size=page, max_num_seqs=seqs, max_num_batched_tokens=budget, num_blocks=pages,
                       enable_chunked_prefill=chunked, max_model_len=max_len)
    cm = CacheManager(page, [GroupSpec(None, pages)], seqs + 1)
    return Scheduler(cfg, cm), cm


def seq(n, max_tokens=8):
    return Sequence(list(range(n)), SamplingParams(max_tokens=max_tokens, ignore_eos=True))


def run_step(sched, batch, finish_after=None):
    """What the engine does after a forward: advance, append one token to rows that ended their tokens."""
    done = []
    for s, n in batch:
        last = s.num_computed + n == s.num_tokens
        sched.advance(s, n)
        if last:
            s.token_ids.append(1)
            if s.num_output_tokens >= s.params.max_tokens:
                sched.finish(s)
                done.append(s)
    return done


def test_three_passes_and_the_budget():
    """Budget 32 with prompts 1/9/40/70: decodes first, then prompts in flight, then admissions
    (inference_engine/scheduler.py:57-102 there)."""
    sched, cm = make(budget=32)
    seqs = [seq(1), seq(9), seq(40), seq(70)]
    for s in seqs:
        sched.add(s)
    b = sched.schedule()
    assert [(s.prompt_len, n) for s, n in b] == [(1, 1), (9, 9), (40, 22)], "strict first come first served, budget 32"
    run_step(sched, b)
    b = sched.schedule()
    # requests 1 and 9 now decode (first), then 40's next portion of 18; 70 is admitted with what is left
    assert [(s.prompt_len, n) for s, n in b] == [(1, 1), (9, 1), (40, 18), (70, 12)]
    assert sum(n for _, n in b) == 32
    run_step(sched, b)
    steps = 2
    while sched.has_work():
        b = sched.schedule()
        assert sum(n for _, n in b) <= 32
        ones = [n == 1 for _, n in b]
        assert ones == sorted(ones, reverse=True), "single tokens come before portions"
        run_step(sched, b)
        steps += 1
        cm.check()
    assert all(s.status is Status.FINISHED and s.num_output_tokens == 8 for s in seqs)
    assert cm.num_free(0) == 39 and not cm.live


def test_without_chunking_a_prompt_waits_for_a_whole_budget():
    sched, _ = make(budget=32, chunked=False)
    a, b_ = seq(20), seq(20)
    sched.add(a)
    sched.add(b_)
    b = sched.schedule()
    assert [(s is a, n) for s, n in b] == [(True, 20)], "the second prompt does not fit whole and is not cut"
    run_step(sched, b)
    b = sched.schedule()
    assert [(s is a, n) for s, n in b] == [(True, 1), (False, 20)]


def test_max_num_seqs_caps_admission():
    sched, _ = make(seqs=2)
    for _ in range(4):
        sched.add(seq(5))
    assert len(sched.schedule()) == 2 and len(sched.running) == 2 and len(sched.waiting) == 2


def test_preemption_takes_the_newest_and_requeues_it_in_front():
    """inference_engine/scheduler.py:38-55 there: victim = running[-1]; its pages go back, it restarts from 0."""
    sched, cm = make(pages=6, budget=64)              # 5 usable pages of 16
    a, b_ = seq(30, max_tokens=40), seq(30, max_tokens=40)
    sched.add(a)
    sched.add(b_)
    run_step(sched, sched.schedule())                  # both admitted: 2 pages each, 1 free
    assert [s.status for s in (a, b_)] == [Status.RUNNING] * 2
    run_step(sched, sched.schedule())                  # token 31, still inside page 2
    run_step(sched, sched.schedule())                  # token 32 -> page boundary next
    assert a.num_tokens == 33
    batch = sched.schedule()                           # a takes the last page, b cannot: b is preempted
    assert sched.num_preemptions == 1 and b_.status is Status.WAITING and b_.num_computed == 0
    assert sched.waiting[0] is b_ and b_.cache is None and b_.num_preemptions == 1
    assert [(s is a, n) for s, n in batch] == [(True, 1)], "no admission in the step that preempted"
    assert b_.num_tokens == 33, "the preempted request keeps its generated tokens"
    cm.check()
    run_step(sched, batch)
    # b comes back only when pages allow: its 33 tokens need 3 pages, 2 are free
    batch = sched.schedule()
    assert all(s is a for s, _ in batch)


def test_requests_that_can_never_fit_raise():
    """The reference spins for ever on these (inference_engine/engine.py:237-238 with scheduler.py:50-54 there)."""
    sched, _ = make(pages=4)                           # 3 usable pages = 48 tokens
    with pytest.raises(RequestTooLarge):
        sched.add(seq(60))
    with pytest.raises(RequestTooLarge):
        sched.add(seq(40, max_tokens=20))
    sched.add(seq(40, max_tokens=8))                   # exactly fits
    run_step(sched, sched.schedule())


def test_a_lone_request_may_use_the_last_pages():
    """The admission watermark keeps room for running requests to grow; with nothing running it
    must not keep a request out that fits (the reference would wait for ever)."""
    sched, _ = make(pages=4, budget=64)
    s = seq(48, max_tokens=0)
    sched.add(s)
    assert [(x is s, n) for x, n in sched.schedule()] == [(True, 48)]


@pytest.mark.parametrize("seed", range(4))
def test_random_workloads_finish_with_all_pages_back(seed):
    rng = random.Random(seed)
    sched, cm = make(pages=rng.choice([8, 12, 30]), budget=rng.choice([16, 48, 2048]), seqs=rng.choice([2, 4, 16]))
    cap = cm.max_tokens_one_request()
    seqs = []
    for _ in range(12):
        n = rng.randint(1, 60)
        seqs.append(seq(n, max_tokens=rng.randint(1, min(30, cap - n))))
    pending = list(seqs)
    steps = 0
    while sched.has_work() or pending:
        if pending and rng.random() < 0.5:
            sched.add(pending.pop(0))
        if not sched.has_work():
            continue
        batch = sched.schedule()
        assert sum(n for _, n in batch) <= sched.cfg.max_num_batched_tokens
        assert len({id(s) for s, _ in batch}) == len(batch), "a request appears once in a step"
        for s, n in batch:
            assert s.status is Status.RUNNING and len(s.cache.tables[0]) * 16 >= s.num_computed + n
        run_step(sched, batch)
        cm.check()
        steps += 1
        assert steps < 5000
    assert all(s.status is Status.FINISHED and s.num_output_tokens == s.params.max_tokens for s in seqs)
    assert cm.num_free(0) == cm.usable_pages(0) and not cm.live


# ------------------------------------------------------------------------------- a step's arrays
def test_a_portion_lengthened_to_a_captured_size_writes_to_the_scratch_page():
    """build_step(pad_portion_to=N): the row's own tokens keep their ids, positions and slots; the padding
    tokens follow at the next positions with id 0, their slots lie in page 0, and the block table names page 0
    beyond the row's own pages."""
    import numpy as np
    import torch
    from types import SimpleNamespace
    from mini_inference_engine_amd.engine.batch import StepArena, StepRow, build_step
    page = 4
    arena = StepArena(32, 4, 16, 1, torch.device("cpu"))
    req = SimpleNamespace(tables=[[7, 3, 9]], state_slot=2)             # positions 0 .. 11
    step = build_step([StepRow(req, [11, 12, 13, 14, 15], 5, [4])], arena, page, pad_portion_to=16, static_context=64)
    assert step.num_tokens == 16 and step.num_rows == 1 and step.num_decode_rows == 0 and step.max_context == 64
    assert step.input_ids.tolist() == [11, 12, 13, 14, 15] + [0] * 11
    assert step.positions.tolist() == list(range(5, 21))
    assert step.logit_rows.tolist() == [4]
    slots = arena.dev_view("slot_mapping0", 16).tolist()
    assert slots[:5] == [3 * page + 1, 3 * page + 2, 3 * page + 3, 9 * page + 0, 9 * page + 1]
    assert all(0 <= s < page for s in slots[5:]), "padding tokens write to page 0"
    table = arena.dev_view("block_tables0", 16).tolist()
    assert table[:3] == [7, 3, 9] and table[3:6] == [0, 0, 0]
    assert step.host["row_context"].tolist() == [21]
    # positions 5 .. 9 need three pages; two are not enough, padding or not
    short = SimpleNamespace(tables=[[7, 3]], state_slot=0)
    with pytest.raises(ValueError, match="pages reserved"):
        build_step([StepRow(short, [1, 2, 3, 4, 5], 5, [])], arena, page, pad_portion_to=16)
    with pytest.raises(ValueError, match="one row"):
        build_step([StepRow(req, [1, 2], 0, []), StepRow(req, [3, 4], 2, [])], arena, page, pad_portion_to=16)
    with pytest.raises(ValueError, match="one row"):
        build_step([StepRow(req, list(range(9)), 0, [])], arena, page, pad_portion_to=8)
