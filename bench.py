"""Headline benchmark: decode tokens/s and prefill tokens/s at the Qwen2.5-0.5B shape, random
weights, synthetic token ids, on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--dtype bfloat16|float32] [--layers L]
                    [--part offline [--requests 300 --offline-prompt 512 --offline-gen 128 --chunked]]
                    [--config CONFIG.json|NAME] (another shape of the architecture; the default is the 0.5B shape)

A "step" is one decode step of the engine (scheduling, metadata upload, the forward pass and greedy
sampling) with a batch of 8 requests, each holding a 2,048-token prompt. One JSON line is printed.
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

# MI355X published peaks
PEAK_HBM_GBS = 8000.0
PEAK_FLOPS = {"bfloat16": 2.5e15, "float32": 157.3e12}


def matmul_params(c: dict) -> int:
    """Parameters of the matrices one token passes through in the layers (no embedding, no head)."""
    h, d = c["hidden_size"], c["hidden_size"] // c["num_attention_heads"]
    q, kv, i = c["num_attention_heads"] * d, c["num_key_value_heads"] * d, c["intermediate_size"]
    return c["num_hidden_layers"] * (h * (q + 2 * kv) + q * h + 3 * h * i)


def decode_bytes(c: dict, batch: int, context: int, elem: int) -> float:
    """Bytes a decode step has to read: every weight it uses once, and the cache of the live requests."""
    h, d = c["hidden_size"], c["hidden_size"] // c["num_attention_heads"]
    q, kv = c["num_attention_heads"] * d, c["num_key_value_heads"] * d
    weights = matmul_params(c) + c["vocab_size"] * h + c["num_hidden_layers"] * (q + 2 * kv + 2 * h) + h
    cache = 2 * c["num_hidden_layers"] * kv * context * batch
    return float((weights + cache) * elem)


def prefill_flops(c: dict, T: int) -> float:
    """Projections 2 * parameters * T, causal attention 2 * T^2 * D * H per layer, one row of logits."""
    d = c["hidden_size"] // c["num_attention_heads"]
    attn = c["num_hidden_layers"] * 2.0 * T * T * d * c["num_attention_heads"]
    return 2.0 * matmul_params(c) * T + attn + 2.0 * c["hidden_size"] * c["vocab_size"]


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
    ap.add_argument("--no-tune", action="store_true", help="keep the library's first choice of matrix-product algorithm")
    ap.add_argument("--skip-points", action="store_true", help="only the headline batch and the prefill")
    ap.add_argument("--part", default="all", choices=["all", "decode", "prefill", "offline"],
                    help="run only the decode steps or only the prefill (for profiling one of them), or an offline "
                         "run: --requests prompts of --offline-prompt tokens submitted at once, --offline-gen tokens each")
    ap.add_argument("--requests", type=int, default=300)
    ap.add_argument("--offline-prompt", type=int, default=512)
    ap.add_argument("--offline-gen", type=int, default=128)
    ap.add_argument("--offline-seqs", type=int, default=128, help="requests running at a time in the offline run")
    ap.add_argument("--chunked", action="store_true", help="offline run: portions of prompts beside decoding requests")
    args = ap.parse_args()
    prompt_len = args.prompt_len
    max_model_len = max(MAX_MODEL_LEN, prompt_len + args.steps + args.warmup + 128)
    if args.gpus != 1:
        print(f"bench.py: this engine runs on one GPU; --gpus {args.gpus} is not supported")
        return 2

    import torch

    from tokenmill_amd import EngineConfig, LLMEngine, SamplingParams
    from tokenmill_amd.engine.loading import load_random_model

    torch.cuda.set_device(0)
    device = torch.device("cuda:0")
    dtype = {"bfloat16": torch.bfloat16, "float32": torch.float32}[args.dtype]
    from tokenmill_amd.config.shapes import read_shape

    shape, shape_name = read_shape(HEADLINE_SHAPE), "Qwen2.5-0.5B shape"
    if args.config:
        shape, shape_name = read_shape(args.config), Path(args.config).stem
    layers_full = shape["num_hidden_layers"]
    if args.layers:
        shape["num_hidden_layers"] = args.layers
    model = load_random_model(shape, seed=0, dtype=dtype, device=device, max_positions=max_model_len)
    elem = 2 if dtype == torch.bfloat16 else 4
    gen = torch.Generator().manual_seed(0)

    def prompts(n):
        return [torch.randint(0, shape["vocab_size"], (prompt_len,), generator=gen).tolist() for _ in range(n)]

    def engine_for(batch):
        pages = batch * (-(-(prompt_len + args.steps + args.warmup + 64) // BLOCK_SIZE)) + 8
        cfg = EngineConfig(dtype=args.dtype, block_size=BLOCK_SIZE, num_blocks=pages, max_model_len=max_model_len,
                           max_num_seqs=max(batch, 1), max_num_batched_tokens=max(prompt_len, batch),
                           watermark=0.0, hip_graphs=not args.no_graphs, tune_gemm=not args.no_tune)
        return LLMEngine(cfg, model=model)

    def time_decode(batch, steps, warmup):
        eng = engine_for(batch)
        sp = SamplingParams(max_tokens=steps + warmup + 8, ignore_eos=True)
        for i, p in enumerate(prompts(batch)):
            eng.add_request(f"d{i}", p, sp)
        while eng.scheduler.queue or any(r.pending > 1 for r in eng.scheduler.live):
            eng.step()                                   # prefills (one prompt a step: budget = 2,048 tokens)
        for _ in range(warmup):
            eng.step()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            outs = eng.step()
            assert len(outs) == batch
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        context = prompt_len + warmup + steps // 2
        for s in list(eng.requests):
            eng.abort_request(s)
        del eng
        return dt / steps, context

    def time_prefill(reps=5):
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
        return statistics.median(times[1:])              # the first run warms up

    def time_offline():
        """All requests at once, as the reference's offline runs do (reference bench/results/results.md:11-18:
        300 requests of 512 prompt and 128 generated tokens); a short run first warms up and captures graphs."""
        per_seq = -(-(args.offline_prompt + args.offline_gen + 1) // BLOCK_SIZE)
        cfg = EngineConfig(dtype=args.dtype, block_size=BLOCK_SIZE, num_blocks=args.offline_seqs * per_seq + 64,
                           max_model_len=max_model_len, max_num_seqs=args.offline_seqs, max_num_batched_tokens=2048,
                           enable_chunked_prefill=args.chunked, hip_graphs=not args.no_graphs,
                           tune_gemm=not args.no_tune)
        eng = LLMEngine(cfg, model=model)
        sp = SamplingParams(max_tokens=args.offline_gen, ignore_eos=True)

        def run(n):
            reqs = [torch.randint(0, shape["vocab_size"], (args.offline_prompt,), generator=gen).tolist() for _ in range(n)]
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            outs = eng.generate(reqs, sp)
            torch.cuda.synchronize()
            assert all(len(o) == args.offline_gen for o in outs)
            return time.perf_counter() - t0
        run(min(args.requests, 2 * args.offline_seqs))
        return run(args.requests)

    if args.part == "offline":
        t = time_offline()
        gen_tokens = args.requests * args.offline_gen
        print(json.dumps({"offline": {"requests": args.requests, "prompt": args.offline_prompt, "gen": args.offline_gen,
                                      "running": args.offline_seqs, "chunked": args.chunked, "s": round(t, 3),
                                      "gen_tok_s": round(gen_tokens / t, 1),
                                      "tok_s": round((gen_tokens + args.requests * args.offline_prompt) / t, 1)}}))
        return 0
    if args.part == "prefill":
        prefill_s = time_prefill()
        print(json.dumps({"prefill": {"value": round(prompt_len / prefill_s, 1), "tokens": prompt_len,
                                      "ms": round(prefill_s * 1e3, 3)}}))
        return 0
    step_s, context = time_decode(args.batch, args.steps, args.warmup)
    value = args.batch / step_s
    if args.part == "decode":
        print(json.dumps({"value": round(value, 1), "ms_per_step": round(step_s * 1e3, 4), "batch": args.batch}))
        return 0
    prefill_s = time_prefill()
    points = {}
    if not args.skip_points:
        for b in (1, 64):
            s, _ = time_decode(b, max(16, args.steps // 2), max(4, args.warmup // 2))
            points[f"decode_b{b}"] = round(b / s, 1)
    nbytes = decode_bytes(shape, args.batch, context, elem)
    achieved = nbytes / step_s / 1e9
    flops = prefill_flops(shape, prompt_len)
    line = {
        "metric": f"decode tok/s at batch {args.batch}, context {prompt_len} ({shape_name}); prefill and batch 1/64 alongside",
        "value": round(value, 1), "unit": "tok/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(step_s * 1e3, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16" if dtype == torch.bfloat16 else "fp32", "data": "synthetic token ids, random weights",
        "config": {"model": shape_name, "layers": shape["num_hidden_layers"], "layers_full": layers_full,
                   "hidden": shape["hidden_size"], "q_heads": shape["num_attention_heads"],
                   "kv_heads": shape["num_key_value_heads"],
                   "head_dim": shape["hidden_size"] // shape["num_attention_heads"],
                   "intermediate": shape["intermediate_size"], "vocab": shape["vocab_size"],
                   "tied": bool(shape.get("tie_word_embeddings", False)),
                   "global_batch": args.batch, "seq_len": prompt_len, "context": context,
                   "max_model_len": max_model_len, "block_size": BLOCK_SIZE, "parallelism": "single GPU",
                   "hip_graphs": not args.no_graphs, "tune_gemm": not args.no_tune, "packed_weights": True},
        "prefill": {"value": round(prompt_len / prefill_s, 1), "tokens": prompt_len, "ms": round(prefill_s * 1e3, 3),
                    "frac": round(flops / prefill_s / PEAK_FLOPS[args.dtype], 4)},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                     "frac": round(achieved / PEAK_HBM_GBS, 4)},
        "points": points,
    }
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    sys.exit(main())
