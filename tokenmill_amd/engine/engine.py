"""The continuous-batching engine: add_request / step / abort_request / generate (reference
src/infer/engine/engine.py:87-281). Every step re-plans the batch, so new requests join at the
next step and finished ones leave at once. Token ids in, token ids out.
"""
from __future__ import annotations

import logging
import random
import time

import torch

from tokenmill_amd.cache.manager import CacheManager
from tokenmill_amd.cache.pool import CachePools
from tokenmill_amd.config.engine_config import EngineConfig
from tokenmill_amd.engine.loading import load_model, resolve_device, resolve_dtype
from tokenmill_amd.engine.runner import ModelRunner, StepEntry
from tokenmill_amd.engine.scheduler import Scheduler
from tokenmill_amd.engine.sequence import RequestOutput, Sequence
from tokenmill_amd.sampling.sampler import Sampler, SamplingParams

log = logging.getLogger("tokenmill_amd.engine")


class RequestRejected(ValueError):
    """The request can never be served (for example, its prompt is longer than max_model_len)."""


def num_cache_pages(cfg: EngineConfig, model, dtype, device, peak_bytes: int) -> int:
    """Pages per layer group: --num-blocks, else --kv-cache-mb, else what is left of
    GPU memory x utilization after weights and peak activations (reference
    src/infer/engine/engine.py:44-84)."""
    if cfg.num_blocks is not None:
        pages = cfg.num_blocks
    else:
        per_page = CachePools.bytes_per_token(model, dtype) * cfg.block_size
        if cfg.kv_cache_mb is not None:
            budget = int(cfg.kv_cache_mb * 2**20)
        else:
            total = torch.cuda.get_device_properties(device).total_memory
            budget = int(total * cfg.gpu_memory_utilization) - peak_bytes
            if budget <= 0:
                raise RuntimeError("no memory left for the cache; lower --max-batched-tokens or raise utilization")
        pages = budget // max(per_page, 1)
        # no request can use more than max_num_seqs * max_model_len tokens
        pages = min(pages, cfg.max_num_seqs * (-(-cfg.max_model_len // cfg.block_size)))
    if pages < 2:
        raise RuntimeError("cache budget too small for the paged pool")
    return int(pages)


TUNE_CANDIDATES = 16        # library algorithms timed per shape with tune_gemm


class LLMEngine:
    def __init__(self, cfg: EngineConfig, model=None):
        self.cfg = cfg
        if model is None:
            self.device = resolve_device(cfg.device)
            self.dtype = resolve_dtype(cfg.dtype)
            model = load_model(cfg.model, self.dtype, self.device, max_positions=cfg.max_model_len,
                               pack_weights=cfg.pack_weights)
        else:
            self.device, self.dtype = model.device, model.dtype
        self.model = model
        if cfg.tune_gemm:
            from tokenmill_amd.hip import ops
            ops.gemm_library_tune(TUNE_CANDIDATES)
        self.eos_ids = set(getattr(model.config, "eos_token_ids", ()) or ())
        peak = self._profile_peak_memory() if (cfg.num_blocks is None and cfg.kv_cache_mb is None) else 0
        pages = num_cache_pages(cfg, model, self.dtype, self.device, peak)
        self.pools = CachePools(model, pages, cfg.block_size, cfg.max_num_seqs, self.dtype, self.device)
        self.cache = CacheManager(self.pools.windows, pages, cfg.block_size, cfg.max_num_seqs, cfg.watermark)
        self.runner = ModelRunner(model, self.pools, max_positions=cfg.max_model_len)
        if cfg.hip_graphs:
            from tokenmill_amd.engine.graphs import DecodeGraphs, StepGraphs
            self.runner.graphs = DecodeGraphs(self.runner, cfg)
            self.runner.step_graphs = StepGraphs(self.runner)
        self.scheduler = Scheduler(cfg, self.cache)
        self.sampler = Sampler(self.device)
        self.seqs: dict[str, Sequence] = {}
        self._rng = random.Random(cfg.seed)
        self._offline_counter = 0
        self.stats = {"steps": 0, "peak_running": 0, "prefill_steps": 0, "decode_steps": 0,
                      "generated_tokens": 0, "busy_time": 0.0}
        log.info("engine ready: %d pages of %d tokens per group (%.0f MiB), dtype %s, device %s", pages,
                 cfg.block_size, self.pools.nbytes / 2**20, self.dtype, self.device)

    def _profile_peak_memory(self) -> int:
        """One dummy step at the largest batch the scheduler will build; returns the peak bytes the
        allocator needed, weights included (reference src/infer/engine/model_runner.py:99-118)."""
        cfg = self.cfg
        n = cfg.max_num_batched_tokens
        seg = min(n, cfg.max_model_len)
        segs = [seg] * (n // seg) + ([n % seg] if n % seg else [])
        pages = sum(-(-s // cfg.block_size) for s in segs)
        pools = CachePools(self.model, pages, cfg.block_size, len(segs), self.dtype, self.device)
        manager = CacheManager(pools.windows, pages, cfg.block_size, len(segs))
        runner = ModelRunner(self.model, pools, max_positions=cfg.max_model_len)
        torch.cuda.synchronize(self.device)
        pool_bytes = pools.nbytes
        torch.cuda.reset_peak_memory_stats(self.device)
        entries = [StepEntry(manager.allocate(f"profile-{i}", s), 0, [0] * s, [s - 1]) for i, s in enumerate(segs)]
        runner.step(entries)
        torch.cuda.synchronize(self.device)
        peak = torch.cuda.max_memory_allocated(self.device) - pool_bytes
        del runner, pools, entries
        torch.cuda.empty_cache()
        return max(peak, 0)

    # --- requests -----------------------------------------------------------------------------------------

    def add_request(self, request_id: str, prompt_ids: list[int], params: SamplingParams,
                    arrival_time: float | None = None) -> Sequence:
        if not prompt_ids:
            raise RequestRejected("prompt is empty")
        if len(prompt_ids) >= self.cfg.max_model_len:
            raise RequestRejected(f"prompt has {len(prompt_ids)} tokens; max_model_len is {self.cfg.max_model_len}")
        if request_id in self.seqs:
            raise RequestRejected(f"duplicate request id {request_id}")
        vocab = self.runner.vocab
        if min(prompt_ids) < 0 or max(prompt_ids) >= vocab:
            raise RequestRejected(f"a prompt token is outside the vocabulary of {vocab}")
        seq = Sequence(request_id, list(prompt_ids), params,
                       arrival_time=time.monotonic() if arrival_time is None else arrival_time)
        seq.sample_seed = params.seed if params.seed is not None else self._rng.getrandbits(62)
        self.seqs[request_id] = seq
        self.scheduler.add(seq)
        return seq

    def abort_request(self, request_id: str, reason: str = "abort") -> RequestOutput | None:
        seq = self.seqs.pop(request_id, None)
        if seq is None:
            return None
        self.scheduler.finish(seq, reason)
        seq.finish_time = time.monotonic()
        return self._output(seq, [])

    def has_unfinished(self) -> bool:
        return self.scheduler.has_unfinished()

    @property
    def num_waiting(self) -> int:
        return len(self.scheduler.waiting)

    # --- one step --------------------------------------------------------------------------------------------

    def step(self) -> list[RequestOutput]:
        outputs: list[RequestOutput] = []
        t0 = time.perf_counter()
        plan = self.scheduler.schedule()
        for seq in plan.ignored:                          # can never fit in the cache
            self.seqs.pop(seq.id, None)
            self.scheduler.finish(seq, "length")
            seq.finish_time = time.monotonic()
            outputs.append(self._output(seq, [], error=None if seq.output_ids else
                                        "prompt does not fit in the KV cache"))
        if plan.empty:
            return outputs
        n_prefill_tokens = plan.num_prefill_tokens
        sampled, tokens = self._execute(plan)
        now = time.monotonic()
        for seq in plan.prefill_seqs:                     # a portion may cover only part of the prompt
            seq.num_computed_tokens += plan.chunk(seq)
        for seq in plan.decode_seqs:
            seq.num_computed_tokens = seq.length
        for seq in plan.seqs:
            self.cache.release_behind_window(seq.cache, seq.num_computed_tokens)
        for seq, tok in zip(sampled, tokens):
            seq.output_ids.append(tok)
            if seq.first_token_time is None:
                seq.first_token_time = now
            reason = self._stop_reason(seq, tok)
            if reason:
                self.scheduler.finish(seq, reason)
                seq.finish_time = now
                self.seqs.pop(seq.id, None)
            outputs.append(self._output(seq, [tok]))
        self._record_step(plan, n_prefill_tokens, time.perf_counter() - t0, len(sampled))
        return outputs

    def _execute(self, plan) -> tuple[list[Sequence], list[int]]:
        """The plan as one batch through the step function; samples one token for every decode and
        for every portion that holds its request's last known token (reference
        src/infer/engine/model_runner.py:76-97)."""
        entries, sampled = [], []
        for seq in plan.prefill_seqs:
            start = seq.num_computed_tokens
            n = plan.chunk(seq)
            done = start + n == seq.length
            entries.append(StepEntry(seq.cache, start, seq.all_token_ids[start:start + n], [n - 1] if done else []))
            if done:
                sampled.append(seq)
        for seq in plan.decode_seqs:
            entries.append(StepEntry(seq.cache, seq.length - 1, [seq.last_token], [0]))
            sampled.append(seq)
        logits = self.runner.step(entries)
        if not sampled:
            return [], []
        tokens = self.sampler.sample(logits, [s.params for s in sampled], [s.sample_seed for s in sampled],
                                     [s.num_output_tokens for s in sampled])
        return sampled, tokens

    def _stop_reason(self, seq: Sequence, tok: int) -> str | None:
        if tok in self.eos_ids and not seq.params.ignore_eos:
            return "stop"
        if seq.num_output_tokens >= seq.params.max_tokens or seq.length >= self.cfg.max_model_len:
            return "length"
        return None

    def _output(self, seq: Sequence, new_tokens: list[int], error: str | None = None) -> RequestOutput:
        return RequestOutput(seq.id, new_tokens, seq.is_finished, seq.finish_reason, seq.num_prompt_tokens,
                             seq.num_output_tokens, seq.arrival_time, seq.first_token_time, seq.finish_time,
                             seq.num_preemptions, error)

    def _record_step(self, plan, n_prefill_tokens: int, step_time: float, n_generated: int) -> None:
        s = self.stats
        s["steps"] += 1
        s["busy_time"] += step_time
        s["prefill_steps" if plan.prefill_seqs else "decode_steps"] += 1
        s["generated_tokens"] += n_generated
        running = len(self.scheduler.running)
        s["peak_running"] = max(s["peak_running"], running)
        if self.cfg.debug_steps:
            log.info("step=%d batch=%d prefill_tokens=%d decode_tokens=%d step_ms=%.2f kv_usage=%.3f "
                     "waiting=%d running=%d preempted=%d", s["steps"], len(plan.seqs), n_prefill_tokens,
                     len(plan.decode_seqs), step_time * 1e3, self.cache.usage(), len(self.scheduler.waiting),
                     running, len(plan.preempted))

    # --- offline helper -----------------------------------------------------------------------------------------

    def generate(self, prompts: list[list[int]], params: SamplingParams | list[SamplingParams]) -> list[list[int]]:
        """Run every prompt to completion through the step loop; returns output token ids in order."""
        plist = params if isinstance(params, list) else [params] * len(prompts)
        seqs = []
        for p, sp in zip(prompts, plist):
            self._offline_counter += 1
            seqs.append(self.add_request(f"offline-{self._offline_counter}", p, sp))
        while self.has_unfinished():
            self.step()
        return [s.output_ids for s in seqs]
