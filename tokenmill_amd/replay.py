"""Trace replay: feed given token ids through a model step by step and write logits.

    bin/trace_run --model DIR --dtype bfloat16|float32 --out DIR --max-tokens N [--block-size P]

Steps are read from standard input, one JSON object a line:

    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}

All entries of a step are one batch. For a step in which something is wanted, ``<out>/<step>.f32``
receives the logits at the wanted places, in the order of the entries and of ``want``, as
little-endian float32 [wanted, vocab]. After every step ``done <step>`` is printed and flushed.
Nothing is sampled. The program drives the engine's own model, step function, cache manager and
kernels (the ones generation uses); it has no forward pass, cache or loader of its own.
"""
from __future__ import annotations

import argparse
import json
import sys
from pathlib import Path

PAGE_SIZE = 16          # tokens per cache page unless --block-size says otherwise (the engine's default)
ROUND_TO = 64           # --max-tokens counts each request's tokens rounded up to this


class ReplaySession:
    """The engine pieces a replay drives: model, cache pools, cache manager and the step function."""

    def __init__(self, model_dir, dtype_name: str, max_tokens: int, max_requests: int = 16,
                 page_size: int = PAGE_SIZE):
        from tokenmill_amd.cache import CacheManager
        from tokenmill_amd.cache.pool import CachePools
        from tokenmill_amd.config.registry import load_config
        from tokenmill_amd.engine.loading import load_model, resolve_device, resolve_dtype
        from tokenmill_amd.engine.runner import ModelRunner
        from tokenmill_amd.hip.library import library

        library()                                # compiles the kernels at the first call of a fresh checkout
        device = resolve_device("auto")
        dtype = resolve_dtype(dtype_name)
        if page_size < 1:
            raise ValueError("--block-size must be at least 1")
        max_tokens = -(-max_tokens // ROUND_TO) * ROUND_TO
        # --max-tokens bounds what all live requests hold together; one request can be no longer than that,
        # nor than the model's own position tables reach
        _, model_config = load_config(model_dir)
        max_positions = min(max_tokens, getattr(model_config, "max_position_embeddings", max_tokens))
        self.model = load_model(model_dir, dtype, device, max_positions=max_positions)
        self.page_size = page_size
        # every request's tokens count rounded up to ROUND_TO; a page that does not divide that may leave
        # one page per request part empty beyond it
        self.num_pages = -(-max_tokens // page_size) + (0 if ROUND_TO % page_size == 0 else max_requests)
        self.pools = CachePools(self.model, self.num_pages, page_size, max_requests, dtype, device)
        self.manager = CacheManager(self.pools.windows, self.num_pages, page_size, max_requests)
        self.runner = ModelRunner(self.model, self.pools, max_positions=max_positions)
        self.lengths: dict[str, int] = {}

    def run_step(self, rec: dict):
        """One line of the trace. Returns float32 logits [wanted, vocab] as a numpy array, or None."""
        import torch

        from tokenmill_amd.engine.runner import StepEntry

        entries = []
        for ent in rec.get("entries", []):
            rid = str(ent["id"])
            tokens = [int(t) for t in ent["tokens"]]
            if not tokens:
                continue
            start = self.lengths.get(rid, 0)
            if rid not in self.manager.live:
                rc = self.manager.allocate(rid, len(tokens))
            else:
                rc = self.manager.live[rid]
                self.manager.append(rc, start + len(tokens))
            entries.append(StepEntry(rc, start, tokens, [int(w) for w in ent.get("want", [])]))
            self.lengths[rid] = start + len(tokens)
        result = None
        if entries:
            logits = self.runner.step(entries)
            if logits.shape[0] > 0:
                result = logits.cpu().numpy()
            else:
                torch.cuda.synchronize()
            for e in entries:
                self.manager.release_behind_window(e.cache, self.lengths[e.cache.request_id])
        for rid in rec.get("end", []):
            rid = str(rid)
            if rid in self.manager.live:
                self.manager.free(self.manager.live[rid])
            self.lengths.pop(rid, None)
        return result


def main(argv=None) -> int:
    p = argparse.ArgumentParser(description="replay a trace of token ids through the engine's step function")
    p.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    p.add_argument("--dtype", required=True, choices=["bfloat16", "float32"])
    p.add_argument("--out", required=True, help="folder for <step>.f32 files")
    p.add_argument("--max-tokens", type=int, required=True,
                   help="most tokens live requests hold at any time (each rounded up to a multiple of 64)")
    p.add_argument("--max-requests", type=int, default=16, help="most requests live at a time")
    p.add_argument("--block-size", type=int, default=PAGE_SIZE, help="tokens per cache page")
    args = p.parse_args(argv)

    print("[trace_run] loading the engine ...", flush=True)
    session = ReplaySession(args.model, args.dtype, args.max_tokens, args.max_requests, args.block_size)
    out_dir = Path(args.out)
    out_dir.mkdir(parents=True, exist_ok=True)
    print(f"[trace_run] ready: {type(session.model.config).__name__}, {args.dtype}, "
          f"{session.num_pages} pages of {session.page_size}", flush=True)
    for line in sys.stdin:
        line = line.strip()
        if not line:
            continue
        rec = json.loads(line)
        logits = session.run_step(rec)
        if logits is not None:
            logits.astype("<f4", copy=False).tofile(out_dir / f"{rec['step']}.f32")
        print(f"done {rec['step']}", flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
