"""One request as the engine keeps it: a single growing token list and a mark of how much of it
is in the cache.

A request is its prompt followed by what it has generated, in one list; ``cached`` counts the
leading tokens whose keys and values lie in the cache. Everything the scheduler needs follows
from the two: ``pending`` tokens still have to run, and a request whose ``pending`` is 1 decodes.
A request that lost its pages goes back to QUEUED with ``cached`` 0: when it is admitted again it
is an ordinary prompt of all its tokens (what the reference calls recompute, reference
src/infer/engine/scheduler.py:230-242), and the index of its next generated token, which keys its
random stream, is unchanged.
"""
from __future__ import annotations

import enum

from tokenmill_amd.cache.manager import RequestCache
from tokenmill_amd.sampling.sampler import SamplingParams


class Phase(enum.Enum):
    QUEUED = "queued"        # holds no pages (new, or evicted: then ``evictions`` > 0)
    LIVE = "live"            # holds pages and a state slot; runs in steps
    DONE = "done"


class Request:
    __slots__ = ("id", "tokens", "n_prompt", "params", "stream_seed", "cached", "cache", "phase", "evictions",
                 "why_done", "error", "t_arrived", "t_first_token", "t_done", "expires")

    def __init__(self, request_id: str, prompt: list[int], params: SamplingParams, stream_seed: int = 0,
                 t_arrived: float = 0.0, expires: bool = True):
        self.id = request_id
        self.tokens: list[int] = list(prompt)
        self.n_prompt = len(self.tokens)
        self.params = params
        self.stream_seed = stream_seed            # with the index of a generated token: its random number
        self.cached = 0
        self.cache: RequestCache | None = None
        self.phase = Phase.QUEUED
        self.evictions = 0
        self.why_done: str | None = None          # stop | length | abort | timeout | error
        self.error: str | None = None
        self.t_arrived = t_arrived
        self.expires = expires                    # False: the engine's request_timeout does not end it
        self.t_first_token: float | None = None
        self.t_done: float | None = None

    def __repr__(self) -> str:
        return f"<Request {self.id} {self.phase.value} {self.n_prompt}+{self.n_generated} tokens, {self.cached} cached>"

    @property
    def n_tokens(self) -> int:
        return len(self.tokens)

    @property
    def n_generated(self) -> int:
        return len(self.tokens) - self.n_prompt

    @property
    def generated(self) -> list[int]:
        return self.tokens[self.n_prompt:]

    @property
    def pending(self) -> int:
        """Tokens that still have to run before the next one can be sampled."""
        return len(self.tokens) - self.cached

    @property
    def done(self) -> bool:
        return self.phase is Phase.DONE


class RequestOutput:
    """What one engine step did for one request (the reference's record of the same name carries the
    same first four facts, reference src/infer/engine/sequence.py:89-105)."""
    __slots__ = ("request_id", "new_token_ids", "finished", "finish_reason", "error", "num_prompt_tokens",
                 "num_output_tokens", "num_preemptions", "arrival_time", "first_token_time", "finish_time")

    def __init__(self, req: Request, new_token_ids: list[int]):
        self.request_id = req.id
        self.new_token_ids = new_token_ids
        self.finished = req.done
        self.finish_reason = req.why_done
        self.error = req.error
        self.num_prompt_tokens = req.n_prompt
        self.num_output_tokens = req.n_generated
        self.num_preemptions = req.evictions
        self.arrival_time, self.first_token_time, self.finish_time = req.t_arrived, req.t_first_token, req.t_done

    def __repr__(self) -> str:
        return (f"RequestOutput({self.request_id!r}, +{self.new_token_ids}, finished={self.finished}, "
                f"reason={self.finish_reason!r}, error={self.error!r})")
