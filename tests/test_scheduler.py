"""The scheduler's decisions, without a model: a small simulation stands in for the engine loop.

What is pinned here are the outcomes the reference's scenarios fix (reference
tests/test_scheduler.py:42-283: 5 tokens on pages of 4 take 2 pages, watermark 10 / 0.2, budget 10
over prompts of 4, 5, 3, portions [7, 7, 6] and [6, 4] -> [2, 6], the newest request is the one
evicted and returns to the queue's front), and this engine's own rules around them.
"""
from __future__ import annotations

import random

import pytest

from tokenmill_amd.cache import CacheManager
from tokenmill_amd.config.engine_config import EngineConfig
from tokenmill_amd.engine.request import Phase, Request
from tokenmill_amd.engine.scheduler import Scheduler, StepPlan
from tokenmill_amd.sampling.sampler import SamplingParams


class Sim:
    """A scheduler over a one-group cache manager, and the part of the engine loop that advances requests."""

    def __init__(self, pages=16, page=4, watermark=0.0, **options):
        cfg = EngineConfig(block_size=page, watermark=watermark, **options)
        self.cache = CacheManager([None], pages, page, num_state_slots=64, watermark=watermark)
        self.sched = Scheduler(cfg, self.cache)
        self.made = 0

    def request(self, n_prompt: int, max_tokens: int = 100, at: float = 0.0) -> Request:
        self.made += 1
        req = Request(f"r{self.made}", list(range(1, n_prompt + 1)), SamplingParams(max_tokens=max_tokens), 0, at)
        self.sched.enqueue(req)
        return req

    def advance(self, plan: StepPlan, token: int = 7) -> StepPlan:
        """What a step does to its requests: the portion is cached, the yielding ones gain a token."""
        for req, entry in zip(plan.owners, plan.entries):
            req.cached += len(entry.tokens)
        for i in plan.yields:
            plan.owners[i].tokens.append(token)
        return plan

    def step(self) -> StepPlan:
        return self.advance(self.sched.plan())

    def pages_of(self, req: Request) -> int:
        return len(req.cache.tables[0]) if req.cache else 0


def test_entries_are_what_the_step_function_takes():
    sim = Sim()
    a = sim.request(5)
    plan = sim.sched.plan()
    (entry,) = plan.entries
    assert entry.cache is a.cache and entry.start == 0 and entry.tokens == [1, 2, 3, 4, 5] and entry.want == [4]
    assert plan.yields == [0] and plan.n_decode == 0 and plan.n_tokens == 5
    sim.advance(plan, token=9)
    plan = sim.sched.plan()
    (entry,) = plan.entries
    assert (entry.start, entry.tokens, entry.want) == (5, [9], [0]) and plan.n_decode == 1


def test_a_prompt_step_then_decode_steps():
    sim = Sim()
    a, b = sim.request(5), sim.request(3)
    plan = sim.step()
    assert plan.prompt_runners == [a, b] and not plan.decoders and plan.n_tokens == 8
    assert sim.pages_of(a) == 2                                 # 5 tokens on pages of 4
    plan = sim.step()
    assert plan.decoders == [a, b] and not plan.prompt_runners


def test_growth_takes_a_page_exactly_at_the_edge():
    sim = Sim()
    a = sim.request(4)
    sim.step()
    assert sim.pages_of(a) == 1 and a.n_tokens == 5             # the 5th token is not cached yet
    sim.step()
    assert sim.pages_of(a) == 2                                 # it is now: the second page appeared
    sim.step()
    assert sim.pages_of(a) == 2


@pytest.mark.parametrize("second, admitted", [(4, 2), (8, 1)])
def test_watermark_holds_pages_back_at_admission(second, admitted):
    sim = Sim(pages=10, watermark=0.2)                          # 2 pages are kept back
    first, other = sim.request(28), sim.request(second)        # 7 pages, then 1 or 2
    plan = sim.sched.plan()
    assert plan.owners == [first, other][:admitted]             # 10 - 7 - 1 = 2 is enough, 10 - 7 - 2 = 1 is not
    assert list(sim.sched.queue) == [first, other][admitted:]


def test_nobody_overtakes_the_head_of_the_queue():
    sim = Sim(pages=4)
    big, small = sim.request(16), sim.request(2)
    assert sim.sched.plan().owners == [big]                     # all 4 pages: small waits
    sim = Sim(pages=4)
    first, blocker, tiny = sim.request(8), sim.request(12), sim.request(1)
    assert sim.sched.plan().owners == [first]                   # tiny would fit, but stands behind blocker
    assert list(sim.sched.queue) == [blocker, tiny]


def test_token_budget_over_whole_prompts():
    sim = Sim(pages=64, max_num_batched_tokens=10)
    a, b, c = sim.request(4), sim.request(5), sim.request(3)
    plan = sim.sched.plan()
    assert plan.owners == [a, b] and plan.n_tokens == 9         # 4 + 5; the 3 would make 12
    assert list(sim.sched.queue) == [c]


def test_a_prompt_beyond_the_budget_runs_alone():
    sim = Sim(pages=64, max_num_batched_tokens=10)
    a, b = sim.request(30), sim.request(2)
    plan = sim.sched.plan()
    assert plan.owners == [a] and plan.n_tokens == 30
    # ... but only as the first of a step: behind another prompt it waits for the next step
    sim = Sim(pages=64, max_num_batched_tokens=10)
    a, b = sim.request(2), sim.request(30)
    assert sim.sched.plan().owners == [a]
    assert sim.sched.plan().owners == [b]


def test_cap_on_live_requests():
    sim = Sim(pages=64, max_num_seqs=2)
    for _ in range(4):
        sim.request(2)
    assert len(sim.sched.plan().owners) == 2 and len(sim.sched.queue) == 2


def test_a_prompt_larger_than_the_pool_is_handed_back():
    sim = Sim(pages=4)
    huge, ok = sim.request(20), sim.request(3)
    plan = sim.sched.plan()
    assert plan.unfit == [huge] and plan.owners == [ok]         # the queue moves on behind it


def test_the_newest_request_is_evicted_and_returns_to_the_front():
    sim = Sim(pages=4)
    old, new = sim.request(4, at=1.0), sim.request(4, at=2.0)
    sim.step()                                                  # both prompts: 2 pages
    late = sim.request(1, at=3.0)
    plan = sim.step()                                           # prompts first: late is admitted, 3 pages
    assert plan.owners == [late]
    # now old and new both want a second page and one is free: the last admitted goes
    plan = sim.sched.plan()
    assert plan.evicted == [late] and sim.sched.live == [old, new]
    assert late.phase is Phase.QUEUED and late.cache is None and late.cached == 0 and late.evictions == 1
    assert sim.sched.queue[0] is late and late.t_arrived == 3.0
    assert plan.decoders == [old, new]
    sim.cache.check_invariants()


def test_an_evicted_request_comes_back_as_a_prompt_of_all_its_tokens():
    sim = Sim(pages=3)
    a, b = sim.request(4), sim.request(4)
    sim.step()
    plan = sim.step()                                           # both need a page, one is free
    assert plan.evicted == [b] and plan.decoders == [a]
    assert b.n_tokens == 5 and b.pending == 5
    sim.sched.retire(a, "stop")
    plan = sim.sched.plan()
    (entry,) = plan.entries
    assert plan.owners == [b] and entry.start == 0 and len(entry.tokens) == 5 and entry.want == [4]
    assert b.n_generated == 1 and sim.sched.evictions == 1      # its next token is still its second


def test_several_evictions_return_in_their_order_of_admission():
    sim = Sim(pages=6, page=2, max_num_seqs=8)
    reqs = [sim.request(2) for _ in range(5)]                   # 5 pages of 6
    sim.step()
    plan = sim.sched.plan()                                     # everyone wants a second page; 1 is free
    assert plan.decoders == reqs[:3]                            # the third can run once the fifth and fourth have gone
    assert plan.evicted == [reqs[4], reqs[3]]                   # newest first
    assert list(sim.sched.queue) == [reqs[3], reqs[4]]          # older one in front again
    sim.cache.check_invariants()


def test_a_lone_request_that_cannot_grow_evicts_itself_and_then_never_fits():
    sim = Sim(pages=1)
    a = sim.request(4)
    sim.step()
    plan = sim.sched.plan()
    assert plan.evicted == [a] and not plan and sim.cache.num_free_pages == 1
    assert sim.sched.plan().unfit == [a]                        # 5 tokens on one page of 4


def test_retire_gives_pages_back_wherever_the_request_stands():
    sim = Sim(pages=8)
    a = sim.request(9)
    sim.sched.plan()
    assert sim.cache.num_free_pages == 5
    sim.sched.retire(a, "abort")
    assert sim.cache.num_free_pages == 8 and a.done and a.why_done == "abort" and not sim.sched.live
    sim.sched.retire(a, "again")                                # a second call changes nothing
    assert a.why_done == "abort"
    b = sim.request(3)
    sim.sched.retire(b, "abort")                                # still queued
    assert not sim.sched.queue and b.done and not sim.sched.busy()
    sim.cache.check_invariants()


def test_nobody_can_join_says_when_the_next_plan_would_admit_nobody():
    """What the engine asks before it queues a decode step ahead of the running one's tokens: with nobody waiting,
    with every slot taken, and with a head of the queue that has to wait for pages, the next plan is the live requests
    again; a free slot and pages for the head, and the policy that counts decode steps while someone waits, need a
    plan of their own."""
    sim = Sim(pages=8, page=4, max_num_seqs=2)
    assert sim.sched.nobody_can_join()
    a, b = sim.request(6), sim.request(6)
    assert not sim.sched.nobody_can_join()               # two slots, pages for the head
    sim.step()
    assert sim.sched.nobody_can_join()                   # nobody waits
    c = sim.request(4)
    assert sim.sched.nobody_can_join()                   # both slots taken
    sim.sched.retire(b, "stop")
    assert not sim.sched.nobody_can_join()               # a slot and 6 free pages for a prompt of one page
    sim.sched.retire(c, "abort")
    d = sim.request(26)                                  # 7 pages: one more than are free while a holds 2
    assert sim.sched.nobody_can_join()
    sim.sched.retire(a, "stop")
    assert not sim.sched.nobody_can_join()
    sim.sched.retire(d, "abort")
    other = Sim(pages=8, page=4, max_num_seqs=1, policy="decode_first")
    other.request(4), other.request(4)
    other.step()
    assert not other.sched.nobody_can_join()             # the slot is taken, and still the plan has to be made: it counts
    mixed = Sim(pages=8, page=4, max_num_seqs=1, enable_chunked_prefill=True)
    mixed.request(4), mixed.request(4)
    mixed.step()
    assert mixed.sched.nobody_can_join()                 # mixed steps admit whenever they can, and now they cannot


def test_decode_first_makes_the_queue_wait():
    sim = Sim(pages=64, policy="decode_first", max_waiting_steps=3)
    a = sim.request(4)
    assert sim.step().owners == [a]                             # nothing is live: the prompt runs
    b = sim.request(4)
    for _ in range(3):
        plan = sim.step()
        assert plan.decoders == [a] and not plan.prompt_runners
    assert sim.step().owners == [b]                             # after 3 decode steps with b waiting
    sim = Sim(pages=64, policy="prefill_first")
    a = sim.request(4)
    sim.step()
    b = sim.request(4)
    assert sim.step().owners == [b]


def test_mixed_steps_cut_a_long_prompt_and_keep_decoding():
    sim = Sim(pages=64, enable_chunked_prefill=True, max_num_batched_tokens=8)
    short = sim.request(3)
    sim.step()
    long = sim.request(20)
    portions = []
    for _ in range(3):
        plan = sim.step()
        assert plan.decoders == [short] and plan.n_tokens <= 8
        portions.append(plan.portion_of(long))
    assert portions == [7, 7, 6]                                # the budget of 8 less one decode
    assert long.n_generated == 1 and long.cached == 20


def test_mixed_steps_share_the_budget_in_queue_order():
    sim = Sim(pages=64, enable_chunked_prefill=True, max_num_batched_tokens=10)
    a, b, c = sim.request(6), sim.request(6), sim.request(6)
    plan = sim.step()
    assert plan.owners == [a, b] and [len(e.tokens) for e in plan.entries] == [6, 4]
    assert plan.yields == [0] and list(sim.sched.queue) == [c]
    plan = sim.step()
    assert plan.decoders == [a] and plan.prompt_runners == [b, c]
    assert [plan.portion_of(b), plan.portion_of(c)] == [2, 6]


def test_mixed_steps_can_evict_a_prompt_that_is_part_way():
    sim = Sim(pages=7, enable_chunked_prefill=True, max_num_batched_tokens=5)
    old = sim.request(4)
    sim.step()
    young = sim.request(20)                                     # 5 pages, 4 tokens a step beside old's decode
    progress = []
    for _ in range(4):
        plan = sim.step()
        assert plan.decoders == [old] and plan.prompt_runners == [young] and plan.portion_of(young) == 4
        progress.append(young.cached)
    assert progress == [4, 8, 12, 16] and sim.cache.num_free_pages == 0 and old.n_tokens == 9
    plan = sim.sched.plan()                                     # old wants a third page
    assert plan.evicted == [young] and plan.decoders == [old] and not plan.prompt_runners
    assert young.cached == 0 and young.phase is Phase.QUEUED and sim.sched.queue[0] is young
    sim.cache.check_invariants()


@pytest.mark.parametrize("mixed", [False, True])
def test_random_traffic_loses_no_page(mixed):
    rng = random.Random(5 + mixed)
    sim = Sim(pages=12, page=4, enable_chunked_prefill=mixed, max_num_batched_tokens=9, max_num_seqs=5)
    reqs = [sim.request(rng.randint(1, 20), max_tokens=rng.randint(1, 12)) for _ in range(30)]
    for _ in range(5000):
        if not sim.sched.busy():
            break
        plan = sim.step()
        if mixed:
            assert plan.n_tokens <= 9
        live = {id(r) for r in sim.sched.live}
        assert all(id(r) in live for r in plan.owners) and len(live) <= 5
        for req in plan.owners:
            if req.n_generated >= req.params.max_tokens:
                sim.sched.retire(req, "length")
        for req in plan.unfit:
            sim.sched.retire(req, "length")
        sim.cache.check_invariants()
    assert not sim.sched.busy() and sim.cache.num_free_pages == 12 and sim.sched.evictions > 0
    assert all(r.done for r in reqs)


def test_padded_step_shapes_hold_every_step_they_stand_for():
    """The shapes that steps are laid out in for graph replay: rows, portions, single tokens and logit rows
    only grow, the rows by at most an eighth beyond the smallest steps, and the tile bound of a shape covers
    every set of portions that fits it (every portion but one may leave a tile part empty)."""
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
