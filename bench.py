"""Headline benchmark: decode tokens/s and prefill tokens/s at the Qwen2.5-0.5B shape, random
weights, synthetic token ids, on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--dtype bfloat16|float32] [--layers L]
                    [--config CONFIG.json|NAME]      another shape of the architecture (7b, 32b, a file)
                    [--part all|decode|prefill|offline|mixed7b|preempt32b]
                    [--part decode --contexts 8192,32768 --batches 8,64]     decode steps over long contexts

A "step" is one decode step of the engine (scheduling, metadata upload, the forward pass and greedy
sampling) with a batch of 8 requests, each holding a 2,048-token prompt. One JSON line is printed:
the decode rate, the step-time histogram, the prefill, decoding at batch 1 and 64 and, at the headline
batch, over contexts of 8,192 and 32,768 tokens (each with the fraction of the HBM peak its step reaches), the step's
roofline fraction, and per operation its GPU time and the share of its own floor it reaches, with
"GPU idle" = wall time - kernel time (what the reference's profiler reports, reference
bench/profile_decode.py:73-82). Bytes and flops come from the model's parts (they state what each
of their operations has to move and do), not from formulas of one architecture.

    --part mixed7b      the 7B shape, context 8,192: prompts of 512 to 4,096 ids arrive into mixed steps
                        (portions of prompts beside decoding requests, budget 2,048), up to 64 at a time
    --part preempt32b   the 32B shape, context 8,192: 64 prompts of 2,048 ids on 8,192 pages of 16, so
                        that growth during decoding evicts requests; reports evictions and tok/s
"""
from __future__ import annotations

import argparse
import json
import statistics
import sys
import time
from pathlib import Path

sys.path.insert(0, str(Path(__file__).resolve().parent))

# the headline configuration: the shipped Qwen2.5-0.5B shape (tokenmill_amd/config/shapes/qwen2.5-0.5b.json)
HEADLINE_SHAPE = "qwen2.5-0.5b"
MAX_MODEL_LEN = 4096
PROMPT_LEN = 2048
BLOCK_SIZE = 16
HISTOGRAM_STEPS = 128            # the step-time histogram is taken over at least this many decode steps
PROFILED_STEPS = 8               # decode steps run under the kernel trace


def percentile(xs: list[float], p: float) -> float:
    s = sorted(xs)
    return s[min(len(s) - 1, int(p * len(s)))]


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=128)
    ap.add_argument("--warmup", type=int, default=16)
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--layers", type=int, default=None, help="fewer layers than the shape has (named in config)")
    ap.add_argument("--prompt-len", type=int, default=PROMPT_LEN,
                    help="tokens of every prompt: the prefill's length and the context the decode steps start from")
    ap.add_argument("--config", default=None, help="a config.json or a shipped shape's name (7b, 32b): run it instead of the 0.5B shape")
    ap.add_argument("--no-graphs", action="store_true", help="launch decode steps kernel by kernel")
    ap.add_argument("--no-pipeline", action="store_true",
                    help="read a decode step's tokens before the next step is queued (as without --pipeline-decode)")
    ap.add_argument("--no-tune", action="store_true", help="keep the library's first choice of matrix-product algorithm")
    ap.add_argument("--tune-every", action="store_true",
                    help="captured shapes also try every algorithm the library holds, not only its heuristic's candidates")
    ap.add_argument("--skip-points", action="store_true", help="only the headline batch and the prefill")
    ap.add_argument("--skip-kernels", action="store_true", help="no per-operation kernel trace")
    ap.add_argument("--part", default="all", choices=["all", "decode", "prefill", "offline", "mixed7b", "preempt32b"],
                    help="all: the headline line. decode / prefill: only that (for profiling one of them). offline: "
                         "--requests prompts of --offline-prompt tokens submitted at once. mixed7b / preempt32b: see above")
    ap.add_argument("--requests", type=int, default=None, help="requests of the offline, mixed7b and preempt32b parts")
    ap.add_argument("--offline-prompt", type=int, default=512)
    ap.add_argument("--offline-gen", type=int, default=128)
    ap.add_argument("--offline-seqs", type=int, default=128, help="requests running at a time in the offline run")
    ap.add_argument("--chunked", action="store_true", help="offline run: portions of prompts beside decoding requests")
    ap.add_argument("--contexts", default=None,
                    help="with --part decode: instead of one batch, a sweep of decode steps over these context lengths (e.g. 8192,32768) "
                         "and the --batches, each with its roofline fraction")
    ap.add_argument("--batches", default="8,64", help="batch sizes of the --contexts sweep")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py: this engine runs on one GPU; --gpus {args.gpus} is not supported")
        return 2
    pipelined = not args.no_pipeline and not args.no_graphs
    if args.part == "mixed7b":
        args.config = args.config or "7b"
    if args.part == "preempt32b":
        args.config = args.config or "32b"
    prompt_len = args.prompt_len
    long_context = args.part in ("mixed7b", "preempt32b")
    max_model_len = 8192 if long_context else max(MAX_MODEL_LEN, prompt_len + args.steps + args.warmup + HISTOGRAM_STEPS + 128)
    # context lengths beyond the headline's, decoded at the headline batch: two more entries of `points` (or, with
    # --contexts, a sweep of its own)
    LONG_POINTS = (8192, 32768)
    sweep = [int(c) for c in args.contexts.split(",")] if args.contexts else []

    import torch

    from tokenmill_amd import EngineConfig, LLMEngine, SamplingParams, profiling
    from tokenmill_amd.config.shapes import read_shape
    from tokenmill_amd.engine.loading import load_random_model

    torch.cuda.set_device(0)
    device = torch.device("cuda:0")
    dtype = {"bfloat16": torch.bfloat16, "float32": torch.float32}[args.dtype]
    shape, shape_name = read_shape(HEADLINE_SHAPE), "Qwen2.5-0.5B shape"
    if args.config:
        shape, shape_name = read_shape(args.config), Path(args.config).stem
    layers_full = shape["num_hidden_layers"]
    if args.layers:
        shape["num_hidden_layers"] = args.layers
    # the position tables reach the longest context any engine of this run allows (each engine has its own limit)
    most_positions = max([max_model_len] + sweep + ([] if args.skip_points or args.part != "all" else list(LONG_POINTS)))
    most_positions = min(most_positions, shape.get("max_position_embeddings", most_positions))
    model = load_random_model(shape, seed=0, dtype=dtype, device=device, max_positions=most_positions)
    gen = torch.Generator().manual_seed(0)
    vocab = shape["vocab_size"]

    def prompts(n, length=None):
        return [torch.randint(0, vocab, (length or prompt_len,), generator=gen).tolist() for _ in range(n)]

    def sizes() -> dict:
        """The shape's sizes for ``config``: the model's own numbers (flat, at most 20 keys with what is added)."""
        heads = shape.get("num_attention_heads")
        return {"model": shape_name, "layers": shape["num_hidden_layers"], "layers_full": layers_full,
                "hidden": shape.get("hidden_size"), "q_heads": heads, "kv_heads": shape.get("num_key_value_heads", heads),
                "head_dim": getattr(model.config, "head_dim", None), "intermediate": shape.get("intermediate_size"),
                "vocab": shape.get("vocab_size"), "tied": bool(shape.get("tie_word_embeddings", False))}

    def engine_for(batch, extra_steps=0, prompt_len=prompt_len, max_model_len=max_model_len):
        pages = batch * (-(-(prompt_len + args.steps + args.warmup + extra_steps + 64) // BLOCK_SIZE)) + 8
        cfg = EngineConfig(dtype=args.dtype, block_size=BLOCK_SIZE, num_blocks=pages, max_model_len=max_model_len,
                           max_num_seqs=max(batch, 1), max_num_batched_tokens=max(prompt_len, batch),
                           watermark=0.0, hip_graphs=not args.no_graphs, tune_gemm=not args.no_tune, tune_gemm_every=args.tune_every and not args.no_tune,
                           pipeline_decode=pipelined)
        return LLMEngine(cfg, model=model)

    def settle(eng):
        """From here on the engine's steps run one at a time: the step in flight is finished and none is queued
        ahead any more (what is measured after this is a single step by itself)."""
        eng.cfg.pipeline_decode = False
        eng.flush()

    def account(fn) -> tuple[float, float]:
        """(bytes, flops) the parts say the device work of ``fn`` has to move and do."""
        with profiling.collect(trace=False) as report:
            fn()
        torch.cuda.synchronize()
        ops = report["ops"].values()
        return sum(o.bytes for o in ops), sum(o.flops for o in ops)

    def eagerly(eng, fn):
        """``fn`` with the engine's graph replay switched off: the same step program runs launch by launch, and
        the library calls the labels' hook around each operation's launches (a replayed graph calls nothing)."""
        runner = eng.runner
        saved = runner.graphs, runner.step_graphs
        runner.graphs = runner.step_graphs = None
        try:
            return fn()
        finally:
            runner.graphs, runner.step_graphs = saved

    def time_decode(batch, steps, warmup, detail=False, context=None):
        """ms per step over exactly ``steps`` steps; with ``detail`` also the histogram over at least
        HISTOGRAM_STEPS steps, the step's bytes, and the kernel trace. ``context``: the requests' length when the
        timed steps end (prompts that much shorter than it), in an engine whose limit is that context; with it the
        step's bytes come back too."""
        extra = (max(0, HISTOGRAM_STEPS - steps) + 2 * PROFILED_STEPS + 4) if detail else 0
        if context is None:
            eng, prompt_tokens = engine_for(batch, extra), prompt_len
        else:
            prompt_tokens = context - steps - warmup - 16
            eng = engine_for(batch, 16, prompt_len=prompt_tokens, max_model_len=context)
        sp = SamplingParams(max_tokens=steps + warmup + extra + 8, ignore_eos=True)
        for i, p in enumerate(prompts(batch, prompt_tokens)):
            eng.add_request(f"d{i}", p, sp)
        while eng.scheduler.queue or any(r.pending > 1 for r in eng.scheduler.live):
            eng.step()                                   # prefills (one prompt a step: budget = 2,048 tokens)
        for _ in range(warmup):
            eng.step()
        eng.step_seconds.clear()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            outs = eng.step()
            assert len(outs) == batch
        torch.cuda.synchronize()
        step_s = (time.perf_counter() - t0) / steps
        out = {"step_s": step_s, "context": prompt_tokens + warmup + steps // 2}
        if context is not None:
            settle(eng)
            out["bytes"], _ = account(lambda: eagerly(eng, eng.step))
        if detail:
            for _ in range(max(0, HISTOGRAM_STEPS - steps)):
                eng.step()
            times = [1e3 * t for t in eng.step_seconds]
            out["step_ms"] = {"p50": round(percentile(times, 0.5), 4), "p90": round(percentile(times, 0.9), 4),
                              "max": round(max(times), 4), "n": len(times)}
            settle(eng)
            out["bytes"], _ = account(lambda: eagerly(eng, eng.step))
            if not args.skip_kernels:
                out.update(trace_decode(eng, step_s))
        for rid in list(eng.requests):
            eng.abort_request(rid)
        del eng
        return out

    def trace_decode(eng, step_s) -> dict:
        """Kernel time of the replayed step (for "GPU idle"), and per operation the GPU time of the same
        step program launched kernel by kernel (what the graph is a recording of), with the share of its
        floor it reaches."""
        with profiling.collect() as replayed:
            for _ in range(PROFILED_STEPS):
                eng.step()
        with profiling.collect() as labelled:
            eagerly(eng, lambda: [eng.step() for _ in range(PROFILED_STEPS)])
        kernel_ms = replayed["kernel_us"] / PROFILED_STEPS / 1e3
        table = {}
        for name, op in sorted(labelled["ops"].items(), key=lambda kv: -kv[1].device_us):
            us = op.device_us / PROFILED_STEPS
            floor = profiling.floor_us(op, args.dtype) / PROFILED_STEPS
            table[f"{name}_us"] = round(us, 1)
            table[f"{name}_frac"] = round(floor / us, 3) if us > 0 else None
        return {"kernels": table, "kernel_ms": round(kernel_ms, 4),
                "gpu_idle_ms": round(max(0.0, step_s * 1e3 - kernel_ms), 4)}

    def time_prefill(reps=5, detail=False):
        eng = engine_for(1)
        times = []
        for r in range(reps + 1):
            p = prompts(1)[0]
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            eng.add_request(f"p{r}", p, SamplingParams(max_tokens=1, ignore_eos=True))
            outs = eng.step()                            # the whole prompt in one step, first token sampled
            torch.cuda.synchronize()
            times.append(time.perf_counter() - t0)
            assert outs and outs[0].finished
        out = {"s": statistics.median(times[1:])}        # the first run warms up

        def one_prompt():
            eng.add_request("pa", prompts(1)[0], SamplingParams(max_tokens=1, ignore_eos=True))
            eng.step()
        _, out["flops"] = account(lambda: eagerly(eng, one_prompt))
        if detail and not args.skip_kernels:
            with profiling.collect() as labelled:
                eagerly(eng, one_prompt)
            table = {}
            for name, op in sorted(labelled["ops"].items(), key=lambda kv: -kv[1].device_us):
                table[f"{name}_us"] = round(op.device_us, 1)
                table[f"{name}_frac"] = round(profiling.floor_us(op, args.dtype) / op.device_us, 3) if op.device_us else None
            out["kernels"] = table
            out["kernel_ms"] = round(labelled["kernel_us"] / 1e3, 3)
        return out

    def serve(eng, reqs, params):
        """Everything submitted at once, run to the end; (seconds, generated tokens)."""
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        outs = eng.generate(reqs, params)
        torch.cuda.synchronize()
        return time.perf_counter() - t0, sum(len(o) for o in outs)

    def time_offline():
        """All requests at once, as the reference's offline runs do (reference bench/results/results.md:11-18:
        300 requests of 512 prompt and 128 generated tokens); a short run first warms up and captures graphs."""
        n = args.requests or 300
        per_seq = -(-(args.offline_prompt + args.offline_gen + 1) // BLOCK_SIZE)
        cfg = EngineConfig(dtype=args.dtype, block_size=BLOCK_SIZE, num_blocks=args.offline_seqs * per_seq + 64,
                           max_model_len=max_model_len, max_num_seqs=args.offline_seqs, max_num_batched_tokens=2048,
                           enable_chunked_prefill=args.chunked, hip_graphs=not args.no_graphs,
                           tune_gemm=not args.no_tune, tune_gemm_every=args.tune_every and not args.no_tune,
                           pipeline_decode=pipelined)
        eng = LLMEngine(cfg, model=model)
        sp = SamplingParams(max_tokens=args.offline_gen, ignore_eos=True)
        serve(eng, prompts(min(n, 2 * args.offline_seqs), args.offline_prompt), sp)
        t, made = serve(eng, prompts(n, args.offline_prompt), sp)
        return {"offline": {"requests": n, "prompt": args.offline_prompt, "gen": args.offline_gen,
                            "running": args.offline_seqs, "chunked": args.chunked, "s": round(t, 3),
                            "gen_tok_s": round(made / t, 1), "tok_s": round((made + n * args.offline_prompt) / t, 1)}}

    def time_mixed():
        """Prompts of 512 to 4,096 ids into mixed steps: portions of prompts beside the decoding requests."""
        n, gen_tokens, seqs, budget = args.requests or 96, 128, 64, 2048
        lengths = torch.randint(512, 4097, (n,), generator=gen).tolist()
        pages = seqs * (-(-(4096 + gen_tokens) // BLOCK_SIZE)) + 64
        cfg = EngineConfig(dtype=args.dtype, block_size=BLOCK_SIZE, num_blocks=pages, max_model_len=max_model_len,
                           max_num_seqs=seqs, max_num_batched_tokens=budget, enable_chunked_prefill=True,
                           hip_graphs=not args.no_graphs, tune_gemm=not args.no_tune, tune_gemm_every=args.tune_every and not args.no_tune,
                           pipeline_decode=pipelined)
        eng = LLMEngine(cfg, model=model)
        sp = SamplingParams(max_tokens=gen_tokens, ignore_eos=True)
        serve(eng, [prompts(1, L)[0] for L in lengths[:8]], SamplingParams(max_tokens=8, ignore_eos=True))    # warm-up
        before = dict(eng.stats)
        eng.step_seconds.clear()
        t, made = serve(eng, [prompts(1, L)[0] for L in lengths], sp)
        s = eng.stats
        times = [1e3 * x for x in eng.step_seconds]
        return {"metric": "generated tok/s, prompts of 512-4,096 ids in mixed steps", "value": round(made / t, 1),
                "unit": "tok/s", "s": round(t, 3), "prompt_tok_s": round(sum(lengths) / t, 1),
                "total_tok_s": round((made + sum(lengths)) / t, 1), "dtype": args.dtype, "data": "synthetic token ids, random weights",
                "steps": s["steps"] - before["steps"], "mixed_steps": s["mixed_steps"] - before["mixed_steps"],
                "step_ms": {"p50": round(percentile(times, 0.5), 3), "p90": round(percentile(times, 0.9), 3), "max": round(max(times), 3)},
                "evictions": eng.scheduler.evictions,
                "config": {**sizes(), "requests": n, "prompt_min": 512, "prompt_max": 4096, "prompt_tokens": sum(lengths),
                           "gen": gen_tokens, "max_num_seqs": seqs, "token_budget": budget, "max_model_len": max_model_len,
                           "block_size": BLOCK_SIZE, "pages": pages}}

    def time_preempt():
        """64 prompts of 2,048 ids on a pool that holds exactly those: every page a decoding request grows
        by has to come from a request that is evicted and recomputed later."""
        n, gen_tokens, pages = args.requests or 64, 64, 8192
        cfg = EngineConfig(dtype=args.dtype, block_size=BLOCK_SIZE, num_blocks=pages, max_model_len=max_model_len,
                           max_num_seqs=n, max_num_batched_tokens=2048, watermark=0.0,
                           hip_graphs=not args.no_graphs, tune_gemm=not args.no_tune, tune_gemm_every=args.tune_every and not args.no_tune,
                           pipeline_decode=pipelined)
        eng = LLMEngine(cfg, model=model)
        sp = SamplingParams(max_tokens=gen_tokens, ignore_eos=True)
        serve(eng, prompts(2), SamplingParams(max_tokens=4, ignore_eos=True))                                 # warm-up
        before = dict(eng.stats)
        t, made = serve(eng, prompts(n), sp)
        s = eng.stats
        eng.cache.check_invariants()
        assert eng.cache.num_free_pages == eng.cache.num_pages
        return {"metric": "generated tok/s with evictions, 64 prompts of 2,048 ids on 8,192 pages", "value": round(made / t, 1),
                "unit": "tok/s", "s": round(t, 3), "evictions": eng.scheduler.evictions, "dtype": args.dtype,
                "data": "synthetic token ids, random weights",
                "steps": s["steps"] - before["steps"], "prompt_steps": s["prompt_steps"] - before["prompt_steps"],
                "decode_steps": s["decode_steps"] - before["decode_steps"],
                "tokens_run": s["tokens_in"] - before["tokens_in"],
                "config": {**sizes(), "requests": n, "prompt": prompt_len, "gen": gen_tokens, "max_num_seqs": n,
                           "token_budget": 2048, "max_model_len": max_model_len, "block_size": BLOCK_SIZE, "pages": pages}}

    if args.part == "offline":
        print(json.dumps(time_offline()))
        return 0
    if args.part == "mixed7b":
        print(json.dumps(time_mixed()))
        return 0
    if args.part == "preempt32b":
        print(json.dumps(time_preempt()))
        return 0
    if args.part == "prefill":
        pre = time_prefill(detail=True)
        print(json.dumps({"prefill": {"value": round(prompt_len / pre["s"], 1), "tokens": prompt_len,
                                      "ms": round(pre["s"] * 1e3, 3),
                                      "frac": round(pre["flops"] / pre["s"] / profiling.PEAK_FLOPS_S[args.dtype], 4),
                                      "kernel_ms": pre.get("kernel_ms"), "kernels": pre.get("kernels")}}))
        return 0
    if args.part == "decode" and sweep:
        rows = {}
        for ctx in sweep:
            for b in [int(v) for v in args.batches.split(",")]:
                d = time_decode(b, args.steps, args.warmup, context=ctx)
                rows[f"b{b}_ctx{ctx}"] = {"tok_s": round(b / d["step_s"], 1), "ms_per_step": round(d["step_s"] * 1e3, 4),
                                          "GB_per_step": round(d["bytes"] / 1e9, 3),
                                          "hbm_frac": round(d["bytes"] / d["step_s"] / profiling.PEAK_HBM_BYTES_S, 4)}
                print(f"b{b}_ctx{ctx}: {rows[f'b{b}_ctx{ctx}']}", file=sys.stderr, flush=True)
        print(json.dumps({"metric": f"decode steps over long contexts ({shape_name})", "dtype": args.dtype, "steps": args.steps,
                          "warmup": args.warmup, "rows": rows}))
        return 0
    dec = time_decode(args.batch, args.steps, args.warmup, detail=True)
    step_s = dec["step_s"]
    value = args.batch / step_s
    if args.part == "decode":
        print(json.dumps({"value": round(value, 1), "ms_per_step": round(step_s * 1e3, 4), "batch": args.batch,
                          "step_ms": dec["step_ms"], "kernel_ms": dec.get("kernel_ms"),
                          "gpu_idle_ms": dec.get("gpu_idle_ms"), "kernels": dec.get("kernels")}))
        return 0
    pre = time_prefill(detail=True)
    points, long_frac = {}, {}
    if not args.skip_points:
        for b in (1, 64):
            d = time_decode(b, max(16, args.steps // 2), max(4, args.warmup // 2))
            points[f"decode_b{b}"] = round(b / d["step_s"], 1)
        for ctx in LONG_POINTS:                          # the headline batch over longer contexts, each against its own roofline
            if ctx > most_positions:
                continue
            d = time_decode(args.batch, 16, 4, context=ctx)
            points[f"decode_b{args.batch}_ctx{ctx}"] = round(args.batch / d["step_s"], 1)
            long_frac[f"ctx{ctx}"] = round(d["bytes"] / d["step_s"] / profiling.PEAK_HBM_BYTES_S, 4)
    achieved = dec["bytes"] / step_s / 1e9
    peak_gbs = profiling.PEAK_HBM_BYTES_S / 1e9
    line = {
        "metric": f"decode tok/s at batch {args.batch}, context {prompt_len} ({shape_name}); prefill and batch 1/64 alongside",
        "value": round(value, 1), "unit": "tok/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(step_s * 1e3, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16" if dtype == torch.bfloat16 else "fp32", "data": "synthetic token ids, random weights",
        "config": {**sizes(), "global_batch": args.batch, "seq_len": prompt_len, "context": dec["context"],
                   "max_model_len": max_model_len, "block_size": BLOCK_SIZE, "parallelism": "single GPU",
                   "hip_graphs": not args.no_graphs, "tune_gemm": ("every" if args.tune_every else True) if not args.no_tune else False, "packed_weights": True, "pipeline_decode": pipelined},
        "prefill": {"value": round(prompt_len / pre["s"], 1), "tokens": prompt_len, "ms": round(pre["s"] * 1e3, 3),
                    "frac": round(pre["flops"] / pre["s"] / profiling.PEAK_FLOPS_S[args.dtype], 4)},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": peak_gbs, "unit": "GB/s",
                     "frac": round(achieved / peak_gbs, 4)},
        "points": points,
        "long_context_hbm_frac": long_frac,
        "step_ms": dec["step_ms"],
        "decode_kernel_ms": dec.get("kernel_ms"), "decode_gpu_idle_ms": dec.get("gpu_idle_ms"),
        "decode_kernels": dec.get("kernels"),
        "prefill_kernel_ms": pre.get("kernel_ms"), "prefill_kernels": pre.get("kernels"),
    }
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    sys.exit(main())
