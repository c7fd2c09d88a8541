"""Plans one step: which requests run how many of their tokens, and who has to give pages back.
Host only; the plan it returns is already the batch the step function takes.

Rules (the reference's decisions, reference src/infer/engine/scheduler.py:95-242; its scenarios are
the vectors of tests/test_scheduler.py):

* The queue is served first come, first served, and nobody overtakes: if the head cannot have its
  pages now, nothing behind it is looked at. A head that could not fit an empty pool is handed
  back as ``unfit``.
* Admission takes pages for every token the request has (prompt and, after an eviction, what it
  had generated), under the cache manager's watermark and the cap on live requests.
* A step runs at most ``max_num_batched_tokens`` tokens. Whole-prompt mode (default): a step is
  prompts only or decodes only; a prompt that does not fit what is left of the budget waits,
  except that the first prompt of a step always runs. Mixed mode (``enable_chunked_prefill``):
  every live request that has one token pending decodes, the budget left goes to prompts that are
  part-way, oldest first, then to the queue; a prompt is cut where the budget ends.
* ``prefill_first`` plans a prompt step whenever the queue's head can be admitted; ``decode_first``
  only when nothing is live or after ``max_waiting_steps`` decode steps with someone waiting.
* Pages run out only when a decoding request crosses a page edge. Then the most recently admitted
  request that this plan has not served yet gives everything back (the request itself if it is the
  last one), and returns to the FRONT of the queue with nothing cached.
"""
from __future__ import annotations

from collections import deque
from dataclasses import dataclass, field

from tokenmill_amd.cache.manager import AllocStatus, CacheManager
from tokenmill_amd.config.engine_config import EngineConfig
from tokenmill_amd.engine.request import Phase, Request
from tokenmill_amd.engine.runner import StepEntry


@dataclass
class StepPlan:
    """A step, as the step function takes it, and what the planning did on the side."""
    entries: list[StepEntry] = field(default_factory=list)     # the n_decode decoding requests first, then prompts
    owners: list[Request] = field(default_factory=list)        # owners[i] runs entries[i]
    yields: list[int] = field(default_factory=list)            # entries whose last row gives the owner's next token
    evicted: list[Request] = field(default_factory=list)       # gave their pages back, newest first
    unfit: list[Request] = field(default_factory=list)         # can never be admitted
    n_decode: int = 0                                          # entries that are one pending token of a live request

    def __bool__(self) -> bool:
        return bool(self.entries)

    @property
    def n_tokens(self) -> int:
        return sum(len(e.tokens) for e in self.entries)

    @property
    def n_prompt_tokens(self) -> int:
        return self.n_tokens - self.n_decode

    @property
    def decoders(self) -> list[Request]:
        return self.owners[:self.n_decode]

    @property
    def prompt_runners(self) -> list[Request]:
        return self.owners[self.n_decode:]

    def portion_of(self, req: Request) -> int:
        """Tokens ``req`` runs in this step (0 if it is not part of it)."""
        return next((len(e.tokens) for e, r in zip(self.entries, self.owners) if r is req), 0)

    def run(self, req: Request, count: int, decode: bool = False) -> None:
        """``req`` runs its next ``count`` tokens; it yields a token if that uses up what it has."""
        start = req.cached
        last = start + count == req.n_tokens
        if last:
            self.yields.append(len(self.entries))
        self.entries.append(StepEntry(req.cache, start, req.tokens[start:start + count], [count - 1] if last else []))
        self.owners.append(req)
        self.n_decode += decode


class Scheduler:
    def __init__(self, cfg: EngineConfig, cache: CacheManager):
        self.cache = cache
        self.token_budget = cfg.max_num_batched_tokens
        self.max_live = cfg.max_num_seqs
        self.mixed = cfg.enable_chunked_prefill
        self.prompts_first = cfg.policy == "prefill_first"
        self.patience = cfg.max_waiting_steps
        self.queue: deque[Request] = deque()
        self.live: list[Request] = []             # in order of admission: the last is the newest
        self.evictions = 0
        self._decode_steps_with_someone_waiting = 0

    # --- coming and going -----------------------------------------------------------------------

    def enqueue(self, req: Request) -> None:
        req.phase = Phase.QUEUED
        self.queue.append(req)

    def busy(self) -> bool:
        return bool(self.queue) or bool(self.live)

    def nobody_can_join(self) -> bool:
        """Would the next plan, made now, admit nobody? True when nobody waits; and, where a plan admits whenever it
        can (mixed steps, or whole prompts first), when every slot of a live request is taken or the head of the queue
        has to wait for pages. (With the policy that lets decode steps run while someone waits, a plan counts those
        steps: then it has to be made.)"""
        if not self.queue:
            return True
        if not self.prompts_first and not self.mixed:
            return False
        if len(self.live) >= self.max_live:
            return True
        return self.cache.allocation_status(self.queue[0].n_tokens) is AllocStatus.LATER

    def retire(self, req: Request, why: str) -> None:
        """The request ends here, wherever it stands; what it holds goes back. Idempotent."""
        if req.phase is Phase.LIVE:
            self.live.remove(req)
            self._give_back(req)
        elif req.phase is Phase.QUEUED and req in self.queue:
            self.queue.remove(req)
        if req.phase is not Phase.DONE:
            req.phase, req.why_done = Phase.DONE, why

    def _give_back(self, req: Request) -> None:
        if req.cache is not None:
            self.cache.free(req.cache)
            req.cache = None

    # --- one plan ---------------------------------------------------------------------------------

    def plan(self) -> StepPlan:
        plan = StepPlan()
        if self.mixed:
            partway = self._plan_decodes(plan, set_aside_prompts=True)
            room = self.token_budget - plan.n_decode
            for req in partway:
                if room <= 0:
                    break
                room -= self._run_portion(plan, req, room)
            self._admit(plan, room, cut=True)
            return plan
        if self.queue and (self.prompts_first or not self.live
                           or self._decode_steps_with_someone_waiting >= self.patience):
            self._admit(plan, self.token_budget, cut=False)
            if plan:
                self._decode_steps_with_someone_waiting = 0
                return plan
        self._plan_decodes(plan)
        if self.queue:
            self._decode_steps_with_someone_waiting += 1
        return plan

    @staticmethod
    def _run_portion(plan: StepPlan, req: Request, room: int) -> int:
        n = min(req.pending, room)
        plan.run(req, n)
        return n

    def _admit(self, plan: StepPlan, room: int, cut: bool) -> None:
        """Heads of the queue become live while they fit. ``cut``: a prompt may run only its first
        ``room`` tokens now; otherwise it runs whole or waits (the step's first prompt always runs)."""
        first = True
        while self.queue and room > 0 and len(self.live) < self.max_live:
            head = self.queue[0]
            fits = self.cache.allocation_status(head.n_tokens)
            if fits is AllocStatus.NEVER:
                plan.unfit.append(self.queue.popleft())
                continue
            if fits is AllocStatus.LATER or (not cut and not first and head.n_tokens > room):
                return
            self.queue.popleft()
            head.cache = self.cache.allocate(head.id, head.n_tokens)
            head.cached = 0
            head.phase = Phase.LIVE
            self.live.append(head)
            count = min(head.pending, room) if cut else head.pending
            plan.run(head, count)
            room -= count
            first = False

    def _plan_decodes(self, plan: StepPlan, set_aside_prompts: bool = False) -> list[Request]:
        """Every live request with one token pending runs it, oldest first, growing by a page where its
        length crosses a page edge. ``live[served:unserved_end]`` are the requests this plan has not
        looked at yet; when a page is missing the last of them is evicted, so the window shrinks
        from both ends and the loop ends when it is empty. Returns the live requests that are still
        inside their prompt (only with ``set_aside_prompts``; they can be evicted until they are
        reached, not after)."""
        live = self.live
        partway: list[Request] = []
        served, unserved_end = 0, len(live)
        while served < unserved_end:
            req = live[served]
            served += 1
            if set_aside_prompts and req.pending > 1:
                partway.append(req)
                continue
            # outside mixed steps a live request has run its whole prompt (a step that fails ends its requests)
            assert req.pending == 1, f"request {req.id} is live with {req.pending} tokens pending"
            grown = self.cache.try_append(req.cache, req.n_tokens)
            while not grown:
                unserved_end -= 1                       # live[unserved_end] is the newest not yet served
                victim = live[unserved_end]
                self._evict(victim, plan)
                if victim is req:
                    break
                grown = self.cache.try_append(req.cache, req.n_tokens)
            if grown:
                plan.run(req, 1, decode=True)
        if unserved_end < len(live):
            # evicted newest first; at the front of the queue they stand oldest first again
            self.queue.extendleft(reversed(live[unserved_end:]))
            del live[unserved_end:]
        return partway

    def _evict(self, req: Request, plan: StepPlan) -> None:
        self._give_back(req)
        req.cached = 0
        req.phase = Phase.QUEUED
        req.evictions += 1
        self.evictions += 1
        plan.evicted.append(req)
