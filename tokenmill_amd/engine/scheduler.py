"""Decides, every step, which requests run a portion of their prompt, which decode one token, and
who is preempted. It never touches the GPU.

The decisions are the reference's (reference src/infer/engine/scheduler.py:29-242):

* FCFS admission without skipping ahead, under the token budget, the cap on running requests and
  the cache manager's watermark; a prompt larger than the whole budget runs alone.
* Not chunked (default): a step is either whole-prompt prefills or decodes. ``prefill_first`` runs
  a prefill step whenever the head of the queue can be admitted; ``decode_first`` only when nothing
  runs or after ``max_waiting_steps`` decode steps.
* Chunked (``enable_chunked_prefill``): every running request that is fully prefilled decodes; the
  budget left goes to prompts already part-way, oldest first, then to new admissions; a prompt is
  cut where the budget ends.
* When pages run out (only decode growth can hit that): the most recently admitted request that
  has not been served this step is preempted, its pages are given back, it goes to the FRONT of the
  waiting queue and is recomputed from its prompt plus what it generated.
"""
from __future__ import annotations

from collections import deque
from dataclasses import dataclass, field

from tokenmill_amd.cache.manager import AllocStatus, CacheManager
from tokenmill_amd.config.engine_config import EngineConfig
from tokenmill_amd.engine.sequence import Sequence, Status


@dataclass
class SchedulerOutput:
    prefill_seqs: list[Sequence] = field(default_factory=list)
    decode_seqs: list[Sequence] = field(default_factory=list)
    preempted: list[Sequence] = field(default_factory=list)
    ignored: list[Sequence] = field(default_factory=list)         # can never fit in the cache
    prefill_chunks: dict = field(default_factory=dict)            # chunked prefill: tokens this step
    num_batched_tokens: int = 0

    def chunk(self, seq: Sequence) -> int:
        """Tokens a prefilling request computes this step."""
        return self.prefill_chunks.get(seq, seq.num_new_tokens)

    @property
    def seqs(self) -> list[Sequence]:
        return self.prefill_seqs + self.decode_seqs

    @property
    def empty(self) -> bool:
        return not self.prefill_seqs and not self.decode_seqs

    @property
    def num_prefill_tokens(self) -> int:
        return sum(self.chunk(s) for s in self.prefill_seqs)


class Scheduler:
    def __init__(self, cfg: EngineConfig, cache: CacheManager):
        self.cfg = cfg
        self.cache = cache
        self.waiting: deque[Sequence] = deque()      # FCFS; preempted requests go back to the front
        self.running: list[Sequence] = []            # admission order, oldest first
        self.num_preemptions = 0
        self._admit_counter = 0
        self._decode_steps_since_prefill = 0

    # --- queues -----------------------------------------------------------------------------------------

    def add(self, seq: Sequence) -> None:
        seq.status = Status.WAITING
        self.waiting.append(seq)

    def has_unfinished(self) -> bool:
        return bool(self.waiting or self.running)

    def finish(self, seq: Sequence, reason: str) -> None:
        """Give back everything the request holds. Safe for a request in any queue."""
        if seq.status == Status.FINISHED:
            return
        if seq in self.running:
            self.running.remove(seq)
            self._release(seq)
        else:
            try:
                self.waiting.remove(seq)
            except ValueError:
                pass
        seq.status = Status.FINISHED
        seq.finish_reason = reason

    def _release(self, seq: Sequence) -> None:
        if seq.cache is not None:
            self.cache.free(seq.cache)
            seq.cache = None

    # --- the plan for one step ------------------------------------------------------------------------------

    def schedule(self) -> SchedulerOutput:
        out = SchedulerOutput()
        if self.cfg.enable_chunked_prefill:
            self._schedule_chunked(out)
            out.num_batched_tokens = len(out.decode_seqs) + out.num_prefill_tokens
            return out
        if self._should_prefill():
            self._schedule_prefills(out)
            if out.prefill_seqs:
                self._decode_steps_since_prefill = 0
                out.num_batched_tokens = out.num_prefill_tokens
                return out
        self._schedule_decodes(self.running, out)
        if self.waiting:
            self._decode_steps_since_prefill += 1
        out.num_batched_tokens = len(out.decode_seqs)
        return out

    def _should_prefill(self) -> bool:
        if not self.waiting:
            return False
        if self.cfg.policy == "prefill_first" or not self.running:
            return True
        return self._decode_steps_since_prefill >= self.cfg.max_waiting_steps

    def _admit(self, seq: Sequence) -> None:
        seq.cache = self.cache.allocate(seq.id, seq.length)      # pages for every token it has, at once
        seq.num_computed_tokens = 0
        seq.status = Status.RUNNING
        seq.admit_order = self._admit_counter
        self._admit_counter += 1
        self.running.append(seq)

    def _head_status(self, out: SchedulerOutput):
        """The head of the queue if it can be admitted now; drops heads that can never fit."""
        while self.waiting:
            seq = self.waiting[0]
            status = self.cache.allocation_status(seq.length)
            if status == AllocStatus.NEVER:
                self.waiting.popleft()
                out.ignored.append(seq)
                continue
            return seq if status == AllocStatus.OK else None        # LATER: nobody skips ahead
        return None

    def _schedule_prefills(self, out: SchedulerOutput) -> None:
        budget = self.cfg.max_num_batched_tokens
        while self.waiting and len(self.running) < self.cfg.max_num_seqs:
            seq = self._head_status(out)
            if seq is None:
                break
            # a prompt that does not fit what is left of the budget waits, unless it is the step's first
            if seq.length > budget and out.prefill_seqs:
                break
            self.waiting.popleft()
            self._admit(seq)
            out.prefill_seqs.append(seq)
            budget -= seq.num_new_tokens
            if budget <= 0:
                break

    def _schedule_decodes(self, candidates: list[Sequence], out: SchedulerOutput,
                          partial: list[Sequence] | None = None) -> None:
        """Each candidate decodes one token. One that crosses a page edge needs a page; if none is
        free the newest request not yet visited this step is preempted until it fits. With
        ``partial`` (chunked mode) requests still inside their prompt are set aside into it instead
        of decoding; until they are visited they can be preempted like any other."""
        queue = sorted(candidates, key=lambda s: s.admit_order)
        try_append, decode_seqs = self.cache.try_append, out.decode_seqs
        i = 0                                               # queue[i:] are the requests not yet visited
        while i < len(queue):
            seq = queue[i]
            i += 1
            if partial is not None and seq.num_new_tokens > 1:
                partial.append(seq)
                continue
            length = seq.length
            while not try_append(seq.cache, length):
                victim = queue.pop() if i < len(queue) else seq
                self._preempt(victim, out)
                if victim is seq:
                    break
            else:
                decode_seqs.append(seq)

    def _schedule_chunked(self, out: SchedulerOutput) -> None:
        budget = self.cfg.max_num_batched_tokens
        # 1. fully prefilled requests decode (a prompt with exactly one uncached token is a decode)
        partial: list[Sequence] = []
        self._schedule_decodes(self.running, out, partial)
        budget -= len(out.decode_seqs)
        # 2. prompts already part-way, oldest first
        for seq in partial:
            if budget <= 0:
                break
            budget -= self._add_chunk(seq, budget, out)
        # 3. new admissions, FCFS, pages for the whole prompt up front
        while self.waiting and budget > 0 and len(self.running) < self.cfg.max_num_seqs:
            seq = self._head_status(out)
            if seq is None:
                break
            self.waiting.popleft()
            self._admit(seq)
            budget -= self._add_chunk(seq, budget, out)

    @staticmethod
    def _add_chunk(seq: Sequence, budget: int, out: SchedulerOutput) -> int:
        out.prefill_seqs.append(seq)
        out.prefill_chunks[seq] = min(seq.num_new_tokens, budget)
        return out.prefill_chunks[seq]

    def _preempt(self, seq: Sequence, out: SchedulerOutput) -> None:
        self.running.remove(seq)
        self._release(seq)
        seq.num_computed_tokens = 0              # recompute prompt + generated tokens on resume
        seq.status = Status.PREEMPTED
        seq.num_preemptions += 1
        self.num_preemptions += 1
        self.waiting.appendleft(seq)             # front of the queue, original arrival time kept
        out.preempted.append(seq)
