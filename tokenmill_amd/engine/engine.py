"""The generation loop. Token ids in, token ids out.

``LLMEngine`` has the reference's five calls (``add_request``, ``step``, ``abort_request``,
``has_unfinished``, ``generate``; reference src/infer/engine/engine.py:87-281). One ``step`` is: the
scheduler plans a batch (which is already the list of entries the step function takes), the step
function returns the logits at the rows that end a request's known tokens, the sampler turns them
into one token each, and the requests are advanced: a request joins at the next plan after it was
added and leaves in the step that ends it.
"""
from __future__ import annotations

import logging
import random
import time
from collections import deque
from dataclasses import dataclass

from tokenmill_amd.cache.manager import CacheManager
from tokenmill_amd.cache.pool import CachePools
from tokenmill_amd.config.engine_config import EngineConfig
from tokenmill_amd.engine.loading import load_model, resolve_device, resolve_dtype
from tokenmill_amd.engine.request import Phase, Request, RequestOutput
from tokenmill_amd.engine.runner import ModelRunner, StepEntry
from tokenmill_amd.engine.scheduler import Scheduler, StepPlan
from tokenmill_amd.engine.sizing import num_cache_pages
from tokenmill_amd.sampling.sampler import Drawn, Sampler, SamplingParams

log = logging.getLogger("tokenmill_amd.engine")

TUNE_CANDIDATES = 16        # library algorithms timed per shape with tune_gemm
STEP_TIMES_KEPT = 8192      # most recent step times kept for a histogram

DOES_NOT_FIT = "prompt does not fit in the KV cache"


class RequestRejected(ValueError):
    """The request can never be served as given (empty, too long, a token outside the vocabulary, an id in use)."""


@dataclass
class _InFlight:
    """A step that has been queued on the GPU and whose tokens have not been read yet."""
    plan: StepPlan
    winners: list[Request]
    drawn: Drawn | None              # None: no entry of the step yields a token
    ahead: bool = False              # queued behind the step before it, before that step's tokens were known


class LLMEngine:
    def __init__(self, cfg: EngineConfig, model=None):
        self.cfg = cfg
        if model is None:
            self.device = resolve_device(cfg.device)
            self.dtype = resolve_dtype(cfg.dtype)
            model = load_model(cfg.model, self.dtype, self.device, max_positions=cfg.max_model_len,
                               pack_weights=cfg.pack_weights)
        else:
            from tokenmill_amd.engine.loading import check_positions
            check_positions(model.config, cfg.max_model_len)
            self.device, self.dtype = model.device, model.dtype
        self.model = model
        self.eos_ids = set(getattr(model.config, "eos_token_ids", ()) or ())
        pages = num_cache_pages(cfg, model, self.dtype, self.device)
        self.pools = CachePools(model, pages, cfg.block_size, cfg.max_num_seqs, self.dtype, self.device)
        self.cache = CacheManager(self.pools.windows, pages, cfg.block_size, cfg.max_num_seqs, cfg.watermark)
        # timing the library's algorithms is this engine's choice: it travels with the engine's own step program
        tune = (TUNE_CANDIDATES, cfg.tune_gemm_every) if cfg.tune_gemm else None
        self.runner = ModelRunner(model, self.pools, max_positions=cfg.max_model_len, tune=tune)
        if cfg.hip_graphs:
            from tokenmill_amd.engine.graphs import DecodeGraphs, StepGraphs
            self.runner.graphs = DecodeGraphs(self.runner, cfg)
            self.runner.step_graphs = StepGraphs(self.runner)
        if cfg.pipeline_decode and not cfg.hip_graphs:
            log.warning("pipeline_decode queues graph replays ahead: without hip_graphs no step is queued ahead")
        self.scheduler = Scheduler(cfg, self.cache)
        self.sampler = Sampler(self.device)
        self.requests: dict[str, Request] = {}           # every request that has not ended
        self._seeds = random.Random(cfg.seed)            # stream seeds of requests that bring none
        self._generate_calls = 0
        self._in_flight: _InFlight | None = None         # with pipeline_decode: the step queued by the call before
        self.stats = {"steps": 0, "prompt_steps": 0, "decode_steps": 0, "mixed_steps": 0, "tokens_out": 0,
                      "tokens_in": 0, "busy_s": 0.0, "peak_live": 0, "steps_ahead": 0, "tokens_dropped": 0}
        self.step_seconds: deque[float] = deque(maxlen=STEP_TIMES_KEPT)
        log.info("engine ready: %d pages of %d tokens per layer group (%.0f MiB), %s on %s", pages, cfg.block_size,
                 self.pools.nbytes / 2**20, self.dtype, self.device)

    # --- requests ---------------------------------------------------------------------------------

    def _check_request(self, request_id: str, prompt_ids: list[int]) -> None:
        vocab, limit = self.runner.vocab, self.cfg.max_model_len
        if request_id in self.requests:
            raise RequestRejected(f"request id {request_id!r} is in use")
        if not prompt_ids:
            raise RequestRejected("the prompt is empty")
        if len(prompt_ids) >= limit:
            raise RequestRejected(f"the prompt has {len(prompt_ids)} tokens and max_model_len is {limit}: "
                                  "no room for a generated token")
        if min(prompt_ids) < 0 or max(prompt_ids) >= vocab:
            raise RequestRejected(f"the prompt holds a token outside the vocabulary of {vocab}")

    def add_request(self, request_id: str, prompt_ids: list[int], params: SamplingParams,
                    arrival_time: float | None = None, expires: bool = True) -> Request:
        """``expires``: False exempts this request from ``request_timeout`` (``generate`` submits a whole batch
        at once, and how long the batch takes is no reason to end the prompts that wait their turn)."""
        self._check_request(request_id, prompt_ids)
        seed = params.seed if params.seed is not None else self._seeds.getrandbits(62)
        req = Request(request_id, prompt_ids, params, seed,
                      time.monotonic() if arrival_time is None else arrival_time, expires=expires)
        self.requests[request_id] = req
        self.scheduler.enqueue(req)
        return req

    def abort_request(self, request_id: str, reason: str = "abort") -> RequestOutput | None:
        req = self.requests.get(request_id)
        if req is None:
            return None
        self._end(req, reason, time.monotonic())
        return RequestOutput(req, [])

    def has_unfinished(self) -> bool:
        return self.scheduler.busy()

    @property
    def num_waiting(self) -> int:
        return len(self.scheduler.queue)

    @property
    def num_running(self) -> int:
        return len(self.scheduler.live)

    def _end(self, req: Request, why: str, now: float, error: str | None = None) -> None:
        self.scheduler.retire(req, why)
        req.t_done, req.error = now, error
        self.requests.pop(req.id, None)

    # --- one step -----------------------------------------------------------------------------------

    def step(self) -> list[RequestOutput]:
        """One step's outputs. With ``pipeline_decode`` the step whose outputs these are was queued by the call
        before, and this call queues the next one behind it before it waits for its tokens."""
        started = time.perf_counter()
        out: list[RequestOutput] = []
        if self.cfg.request_timeout:
            # a request that has been here too long ends before the step is planned, queued or live,
            # and gives its pages back (reference src/infer/engine/engine.py:169-170,213-216)
            too_old = time.monotonic() - self.cfg.request_timeout
            for req in [r for r in self.requests.values() if r.expires and r.t_arrived < too_old]:
                self._end(req, "timeout", time.monotonic())
                out.append(RequestOutput(req, []))
        flight, self._in_flight = self._in_flight, None
        if flight is None:
            plan = self.scheduler.plan()
            for req in plan.unfit:
                # an evicted request that has grown past the pool ends with what it has; a fresh one with an error
                self._end(req, "length", time.monotonic(), None if req.n_generated else DOES_NOT_FIT)
                out.append(RequestOutput(req, []))
            if not plan:
                return out
            flight = self._launch(plan)
        ahead = self._launch_ahead(flight) if self.cfg.pipeline_decode else None
        try:
            out.extend(self._finish(flight, started))
        except BaseException:
            if ahead is not None:                     # queued behind a step that failed: what it computed is void
                self._fail(ahead.plan, RuntimeError("the step before this one failed"))
            raise
        self._in_flight = ahead
        return out

    def flush(self) -> list[RequestOutput]:
        """The outputs of the step that is in flight (with ``pipeline_decode``: queued by the last call), if any, without
        queueing another behind it: after this the GPU holds no work of the engine's."""
        flight, self._in_flight = self._in_flight, None
        return self._finish(flight, time.perf_counter()) if flight is not None else []

    def _fail(self, plan: StepPlan, e: BaseException) -> None:
        """The step did not run to its end, so what the cache holds for its requests is unknown: they end
        here with the error and give their pages back (the reference's loop ends every request in
        flight with the error and goes on serving, reference src/infer/engine/engine.py:342-349).
        Requests that were not part of the step are untouched."""
        now = time.monotonic()
        for req in dict.fromkeys(plan.owners):
            if req.phase is Phase.LIVE:
                self._end(req, "error", now, f"{type(e).__name__}: {e}")

    def _launch(self, plan: StepPlan) -> _InFlight:
        """Queue the plan's step and the sampling of its tokens; nothing is waited for."""
        winners = [plan.owners[i] for i in plan.yields]
        try:
            logits = self.runner.step(plan.entries)
            drawn = self.sampler.start(logits, [r.params for r in winners], [r.stream_seed for r in winners],
                                       [r.n_generated for r in winners]) if winners else None
        except Exception as e:
            self._fail(plan, e)
            raise
        return _InFlight(plan, winners, drawn)

    def _launch_ahead(self, flight: _InFlight) -> _InFlight | None:
        """While ``flight`` runs: queue the step after it, if that step is known without ``flight``'s tokens but for
        their values. That is so when ``flight`` is a decode step of requests that all go on unless they meet an
        end-of-sequence token (none reaches its ``max_tokens`` or the model's length with this token), nobody who waits
        could be admitted now, and every request has a page for its next position: then the next step is the same requests,
        one position on, and the ids go from the sampler's output to the step's input on the device. A request that
        does end at an end-of-sequence token has then run one token too many; it is dropped when that step's tokens
        are read. None: the next step is planned the usual way, after ``flight``'s tokens."""
        plan = flight.plan
        n = len(plan.entries)
        if (flight.drawn is None or plan.n_decode != n or len(plan.yields) != n or self.runner.graphs is None
                or len(self.scheduler.live) != n or not self.scheduler.nobody_can_join()):
            return None
        limit = self.cfg.max_model_len
        for req in plan.owners:
            if (req.phase is not Phase.LIVE or req.n_generated + 1 >= req.params.max_tokens or req.n_tokens + 1 >= limit):
                return None
        for req in plan.owners:
            if not self.cache.try_append(req.cache, req.n_tokens + 1):
                return None
        # flight's token is not in req.tokens yet: it will sit at position req.cached + 1 = req.n_tokens
        entries = [StepEntry(req.cache, req.cached + 1, [0], [0]) for req in plan.owners]
        try:
            logits = self.runner.step_behind(entries, flight.drawn.device)
            if logits is None:
                return None
            owners = list(plan.owners)
            drawn = self.sampler.start(logits, [r.params for r in owners], [r.stream_seed for r in owners],
                                       [r.n_generated + 1 for r in owners])
        except Exception as e:                        # nothing of it counts; the usual way takes over
            log.warning("no step queued ahead (%s: %s)", type(e).__name__, e)
            return None
        self.stats["steps_ahead"] += 1
        return _InFlight(StepPlan(entries=entries, owners=owners, yields=list(range(n)), n_decode=n), owners, drawn,
                         ahead=True)

    def _finish(self, flight: _InFlight, started: float) -> list[RequestOutput]:
        """Wait for the step's tokens and advance its requests. A request that ended since the step was queued (an
        end-of-sequence token in the step before a step queued ahead, an abort, a timeout) is passed over: its
        row's token is dropped."""
        plan, out = flight.plan, []
        try:
            tokens = flight.drawn.tokens() if flight.drawn is not None else []
        except Exception as e:
            self._fail(plan, e)
            raise
        now = time.monotonic()
        release = self.cache.release_behind_window
        for req, entry in zip(plan.owners, plan.entries):
            if req.phase is Phase.LIVE and req.cache is entry.cache:
                req.cached += len(entry.tokens)
                release(req.cache, req.cached)
        n_out = 0
        for req, token in zip(flight.winners, tokens):
            if req.phase is not Phase.LIVE:
                self.stats["tokens_dropped"] += 1
                continue
            req.tokens.append(token)
            n_out += 1
            if req.t_first_token is None:
                req.t_first_token = now
            why = self._why_stop(req, token)
            if why is not None:
                self._end(req, why, now)
            out.append(RequestOutput(req, [token]))
        self._account(plan, n_out, time.perf_counter() - started)
        return out

    def _why_stop(self, req: Request, token: int) -> str | None:
        """"stop" at an end-of-sequence token (which stays in the output), "length" at the request's or the
        model's limit (reference src/infer/engine/engine.py:206-216)."""
        if token in self.eos_ids and not req.params.ignore_eos:
            return "stop"
        if req.n_generated >= req.params.max_tokens or req.n_tokens >= self.cfg.max_model_len:
            return "length"
        return None

    def _account(self, plan: StepPlan, n_out: int, seconds: float) -> None:
        s = self.stats
        n_decode, n_prompt = plan.n_decode, plan.n_prompt_tokens
        s["steps"] += 1
        s["mixed_steps" if n_decode and n_prompt else ("decode_steps" if n_decode else "prompt_steps")] += 1
        s["tokens_out"] += n_out
        s["tokens_in"] += n_prompt + n_decode
        s["busy_s"] += seconds
        s["peak_live"] = max(s["peak_live"], len(plan.entries))
        self.step_seconds.append(seconds)
        if self.cfg.debug_steps:
            log.info("step %d: %d entries (%d prompt tokens + %d decodes) in %.2f ms; cache %.1f%% used; "
                     "%d queued, %d live, %d evicted", s["steps"], len(plan.entries), n_prompt, n_decode,
                     seconds * 1e3, 100 * self.cache.usage(), len(self.scheduler.queue), len(self.scheduler.live),
                     len(plan.evicted))

    # --- all at once ---------------------------------------------------------------------------------

    def generate(self, prompts: list[list[int]], params: SamplingParams | list[SamplingParams]) -> list[list[int]]:
        """Every prompt to its end through the step loop; the generated ids, in the prompts' order."""
        each = params if isinstance(params, list) else [params] * len(prompts)
        if len(each) != len(prompts):
            raise ValueError(f"{len(prompts)} prompts but {len(each)} sampling parameters")
        self._generate_calls += 1
        names = [f"generate-{self._generate_calls}-{i}" for i in range(len(prompts))]
        for name, p in zip(names, prompts):          # all or none: a prompt that is refused leaves nothing queued
            self._check_request(name, p)
        # all of them arrive now and wait their turn, so none of them expires; requests that came through
        # add_request keep their timeout
        reqs = [self.add_request(name, p, sp, expires=False) for name, p, sp in zip(names, prompts, each)]
        try:
            while any(not r.done for r in reqs):
                self.step()
        except BaseException:
            for r in reqs:                           # what the failed step did not end gives its pages back too
                self.abort_request(r.id)
            raise
        return [r.generated for r in reqs]
