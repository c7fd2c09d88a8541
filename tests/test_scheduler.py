"""Scheduler decisions with fake requests and no model: admission, budgets, preemption, policies.

The scenarios and their expected outcomes are the reference's (reference
tests/test_scheduler.py:42-283), run against this engine's scheduler and cache manager.
"""
from __future__ import annotations

from tokenmill_amd.cache import CacheManager
from tokenmill_amd.config.engine_config import EngineConfig
from tokenmill_amd.engine.scheduler import Scheduler
from tokenmill_amd.engine.sequence import Sequence, Status
from tokenmill_amd.sampling.sampler import SamplingParams


def make(num_blocks=16, block_size=4, watermark=0.0, **cfg_kw):
    cfg = EngineConfig(block_size=block_size, watermark=watermark, **cfg_kw)
    cache = CacheManager([None], num_blocks, block_size, num_state_slots=64, watermark=watermark)
    return Scheduler(cfg, cache), cache


_n = 0


def seq(prompt_len, max_tokens=100, arrival=0.0) -> Sequence:
    global _n
    _n += 1
    return Sequence(f"s{_n}", list(range(1, prompt_len + 1)), SamplingParams(max_tokens=max_tokens),
                    arrival_time=arrival)


def pages(s: Sequence) -> int:
    return len(s.cache.tables[0]) if s.cache else 0


def run_step(sched, plan, token=7):
    """What the engine does after a forward pass: mark tokens computed, append one token each."""
    for s in plan.seqs:
        s.num_computed_tokens = s.length
        s.output_ids.append(token)


def run_chunked_step(sched, plan, token=7):
    for s in plan.prefill_seqs:
        s.num_computed_tokens += plan.chunk(s)
    for s in plan.decode_seqs:
        s.num_computed_tokens = s.length
    for s in plan.seqs:
        if s.num_computed_tokens == s.length:
            s.output_ids.append(token)


def test_prefill_then_decode():
    sched, cache = make()
    a, b = seq(5), seq(3)
    sched.add(a), sched.add(b)
    plan = sched.schedule()
    assert plan.prefill_seqs == [a, b] and not plan.decode_seqs
    assert plan.num_batched_tokens == 8
    assert pages(a) == 2                                        # ceil(5 / 4)
    run_step(sched, plan)
    plan = sched.schedule()
    assert plan.decode_seqs == [a, b] and not plan.prefill_seqs


def test_admission_respects_watermark():
    sched, cache = make(num_blocks=10, watermark=0.2)          # 2 pages held back
    a, b = seq(4 * 7), seq(4)
    sched.add(a), sched.add(b)
    assert sched.schedule().prefill_seqs == [a, b]              # 10 - 7 = 3 >= 2 ok; then 3 - 1 = 2 >= 2 ok
    sched2, _ = make(num_blocks=10, watermark=0.2)
    c, d = seq(4 * 7), seq(4 * 2)
    sched2.add(c), sched2.add(d)
    assert sched2.schedule().prefill_seqs == [c]                # d would leave 1 < 2 free
    assert list(sched2.waiting) == [d]


def test_admission_is_fcfs():
    sched, _ = make(num_blocks=4)
    big, small = seq(4 * 4), seq(2)
    sched.add(big), sched.add(small)
    assert sched.schedule().prefill_seqs == [big]               # small waits behind big (no skipping)
    sched2, _ = make(num_blocks=4)
    first, blocker, tiny = seq(4 * 2), seq(4 * 3), seq(1)
    for x in (first, blocker, tiny):
        sched2.add(x)
    assert sched2.schedule().prefill_seqs == [first]            # tiny would fit but waits behind blocker
    assert list(sched2.waiting) == [blocker, tiny]


def test_token_budget_holds():
    sched, _ = make(num_blocks=64, max_num_batched_tokens=10)
    a, b, c = seq(4), seq(5), seq(3)
    for s in (a, b, c):
        sched.add(s)
    plan = sched.schedule()
    assert plan.prefill_seqs == [a, b] and plan.num_batched_tokens == 9
    assert list(sched.waiting) == [c]


def test_prompt_bigger_than_budget_runs_alone():
    sched, _ = make(num_blocks=64, max_num_batched_tokens=10)
    a, b = seq(30), seq(2)
    sched.add(a), sched.add(b)
    assert sched.schedule().prefill_seqs == [a]


def test_max_num_seqs():
    sched, _ = make(num_blocks=64, max_num_seqs=2)
    for _ in range(4):
        sched.add(seq(2))
    assert len(sched.schedule().prefill_seqs) == 2


def test_never_fits_is_ignored():
    sched, _ = make(num_blocks=4)
    huge = seq(4 * 5)
    sched.add(huge)
    plan = sched.schedule()
    assert plan.ignored == [huge] and plan.empty


def test_growth_allocates_one_page_at_the_edge():
    sched, cache = make(num_blocks=16)
    a = seq(4)
    sched.add(a)
    run_step(sched, sched.schedule())                           # length 5 now: needs a 2nd page
    assert pages(a) == 1
    plan = sched.schedule()
    assert plan.decode_seqs == [a] and pages(a) == 2
    run_step(sched, plan)                                       # length 6: still 2 pages
    sched.schedule()
    assert pages(a) == 2


def test_preemption_picks_newest_and_requeues_at_front():
    sched, cache = make(num_blocks=4)
    old, new = seq(4, arrival=1.0), seq(4, arrival=2.0)
    later = seq(1, arrival=3.0)
    sched.add(old), sched.add(new)
    run_step(sched, sched.schedule())                           # both prefilled: 2 pages used
    sched.add(later)
    plan = sched.schedule()                                     # later prefills (1 page): 3 used
    assert plan.prefill_seqs == [later]
    run_step(sched, plan)
    # Decode: old and new each need a 2nd page, later needs none. Only 1 page is free.
    plan = sched.schedule()
    assert plan.preempted == [later]
    assert later.admit_order == max(s.admit_order for s in (old, new, later))     # most recently admitted
    assert later.status == Status.PREEMPTED and later.cache is None
    assert sched.waiting[0] is later                            # front of the queue
    assert old in plan.decode_seqs
    cache.check_invariants()


def test_preempted_request_resumes_with_all_tokens():
    sched, cache = make(num_blocks=3)
    a, b = seq(4), seq(4)
    sched.add(a), sched.add(b)
    run_step(sched, sched.schedule())
    plan = sched.schedule()                                     # both need a 2nd page; 1 free
    assert plan.preempted == [b] and plan.decode_seqs == [a]
    assert b.num_computed_tokens == 0 and b.length == 5
    run_step(sched, plan)
    sched.finish(a, "stop")                                     # a leaves; b can come back
    plan = sched.schedule()
    assert plan.prefill_seqs == [b]
    assert b.num_new_tokens == 5                                # prompt + generated token recomputed
    assert b.arrival_time == 0.0 and b.num_preemptions == 1 and sched.num_preemptions == 1


def test_a_request_alone_that_cannot_grow_preempts_itself():
    sched, cache = make(num_blocks=1)
    a = seq(4)
    sched.add(a)
    run_step(sched, sched.schedule())
    plan = sched.schedule()
    assert plan.preempted == [a] and plan.empty and cache.num_free_pages == 1
    plan = sched.schedule()                                     # 5 tokens need 2 pages of 1: never
    assert plan.ignored == [a]


def test_finish_frees_pages():
    sched, cache = make(num_blocks=8)
    a = seq(9)
    sched.add(a)
    sched.schedule()
    assert cache.num_free_pages == 5
    sched.finish(a, "abort")
    assert cache.num_free_pages == 8 and a.status == Status.FINISHED and not sched.running
    sched.finish(a, "abort")                                    # safe to call again
    b = seq(3)
    sched.add(b)
    sched.finish(b, "abort")                                    # and for a request still waiting
    assert not sched.waiting and b.finish_reason == "abort"
    cache.check_invariants()


def test_decode_first_defers_prefill():
    sched, _ = make(num_blocks=64, policy="decode_first", max_waiting_steps=3)
    a = seq(4)
    sched.add(a)
    run_step(sched, sched.schedule())                           # nothing running: prefill allowed
    b = seq(4)
    sched.add(b)
    for _ in range(3):
        plan = sched.schedule()
        assert plan.decode_seqs == [a] and not plan.prefill_seqs
        run_step(sched, plan)
    assert sched.schedule().prefill_seqs == [b]                 # waited max_waiting_steps decode steps


def test_prefill_first_admits_immediately():
    sched, _ = make(num_blocks=64, policy="prefill_first")
    a = seq(4)
    sched.add(a)
    run_step(sched, sched.schedule())
    b = seq(4)
    sched.add(b)
    assert sched.schedule().prefill_seqs == [b]


def test_chunked_prefill_splits_long_prompt_and_keeps_decoding():
    sched, _ = make(num_blocks=64, enable_chunked_prefill=True, max_num_batched_tokens=8)
    short = seq(3)
    sched.add(short)
    run_chunked_step(sched, sched.schedule())                   # short prompt prefilled whole
    long = seq(20)
    sched.add(long)
    chunks = []
    for _ in range(3):
        plan = sched.schedule()
        assert short in plan.decode_seqs                        # the running stream never stalls
        assert plan.num_batched_tokens <= 8
        if long in plan.prefill_seqs:
            chunks.append(plan.chunk(long))
        run_chunked_step(sched, plan)
    assert chunks == [7, 7, 6]                                  # 8-token budget minus 1 decode each step
    assert long.num_output_tokens == 1 and long.num_computed_tokens == 20


def test_chunked_prefill_budget_shared_fcfs():
    sched, _ = make(num_blocks=64, enable_chunked_prefill=True, max_num_batched_tokens=10)
    a, b, c = seq(6), seq(6), seq(6)
    for s in (a, b, c):
        sched.add(s)
    plan = sched.schedule()
    assert [plan.chunk(s) for s in plan.prefill_seqs] == [6, 4]  # a whole, b partly; c waits
    assert list(sched.waiting) == [c]
    run_chunked_step(sched, plan)
    plan = sched.schedule()                                     # a decodes, b finishes, c starts
    assert plan.decode_seqs == [a] and plan.prefill_seqs[:1] == [b] and plan.chunk(b) == 2
    assert plan.prefill_seqs[1:] == [c] and plan.chunk(c) == 6


def test_chunked_preemption_can_take_a_prompt_that_is_part_way():
    sched, cache = make(num_blocks=7, enable_chunked_prefill=True, max_num_batched_tokens=5)
    old = seq(4)
    sched.add(old)
    run_chunked_step(sched, sched.schedule())                   # old: 1 page, length 5
    young = seq(20)                                             # 5 pages, prefilled 4 tokens a step
    sched.add(young)
    seen = []
    for _ in range(4):                                          # steps 2..5: old decodes, young advances
        plan = sched.schedule()
        assert plan.decode_seqs == [old] and plan.prefill_seqs == [young] and plan.chunk(young) == 4
        run_chunked_step(sched, plan)
        seen.append(young.num_computed_tokens)
    assert seen == [4, 8, 12, 16] and cache.num_free_pages == 0 and old.length == 9
    plan = sched.schedule()                                     # old needs a 3rd page: the newest goes, part-way
    assert plan.preempted == [young] and plan.decode_seqs == [old] and not plan.prefill_seqs
    assert young.num_computed_tokens == 0 and young.status == Status.PREEMPTED and sched.waiting[0] is young
    cache.check_invariants()


def test_every_page_is_back_after_random_traffic():
    import random
    rng = random.Random(0)
    sched, cache = make(num_blocks=12, block_size=4, enable_chunked_prefill=True, max_num_batched_tokens=9,
                        max_num_seqs=5)
    seqs = [seq(rng.randint(1, 20), max_tokens=rng.randint(1, 12)) for _ in range(30)]
    for s in seqs:
        sched.add(s)
    steps = 0
    while sched.has_unfinished() and steps < 5000:
        plan = sched.schedule()
        assert plan.num_batched_tokens <= 9
        run_chunked_step(sched, plan)
        for s in plan.seqs:
            if s.num_output_tokens >= s.params.max_tokens:
                sched.finish(s, "length")
        for s in plan.ignored:
            sched.finish(s, "length")
        cache.check_invariants()
        steps += 1
    assert not sched.has_unfinished() and cache.num_free_pages == 12 and sched.num_preemptions > 0


def test_padded_step_shapes_hold_every_step_they_stand_for():
    """The shapes that steps are laid out in for graph replay: rows, portions, single tokens and logit rows
    only grow, the rows by at most an eighth beyond the smallest steps, and the tile bound of a shape covers
    every set of portions that fits it (every portion but one may leave a tile part empty)."""
    import random
    from types import SimpleNamespace

    from tokenmill_amd.engine.graphs import StepGraphs
    from tokenmill_amd.engine.runner import ModelRunner

    rng = random.Random(0)
    for _ in range(20000):
        portions = [rng.choice([2, 3, 15, 16, 17, 18, 31, 32, 33, rng.randint(2, 300)]) for _ in range(rng.randint(1, 12))]
        singles = rng.randint(0, 40)
        entries = [SimpleNamespace(tokens=[0] * n, want=[n - 1] if rng.random() < 0.5 else []) for n in portions]
        entries += [SimpleNamespace(tokens=[0], want=[0]) for _ in range(singles)]
        rows, P, ND, R = StepGraphs.padded_shape(entries)
        total = sum(portions)
        assert rows >= total and rows % 32 == 0 and (rows - total < 32 or rows <= total * 1.125)
        assert P >= len(portions) and ND >= singles and R >= sum(len(e.want) for e in entries)
        assert P < 2 * len(portions) and (ND < 2 * singles or singles == 0)
        assert sum(-(-n // 16) for n in portions) <= ModelRunner.padded_tiles(rows, P)
    assert ModelRunner.padded_tiles(2048, 1) == 128
