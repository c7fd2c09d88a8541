"""Offline generation from the command line, in the manner of the reference's one CLI entry point
(``python -m infer.serve`` with the engine flags, reference src/infer/serve.py:1-44): the same
engine flags, plus where the prompts come from and how to sample.

    python -m tokenmill_amd.generate --model DIR --prompt-ids "1,2,3;4,5" --max-tokens 16
    python -m tokenmill_amd.generate --model DIR --prompt-lens 5,17,33 --prompt-seed 0 --temperature 0.8
    python -m tokenmill_amd.generate --random CONFIG.json --weights-seed 1 --prompt-lens 64 --max-tokens 32

``--random`` takes a config.json (or a folder holding one) or the name of a shipped shape (0.5b, 7b, 32b,
tiny-a, tiny-b) and draws the weights on the device from ``--weights-seed`` instead of reading a checkpoint.

Token ids in, token ids out (one JSON line per prompt).
"""
from __future__ import annotations

import argparse
import json
import logging
import sys

from tokenmill_amd.config.engine_config import add_engine_args, engine_config_from_args


def main(argv=None) -> int:
    parser = argparse.ArgumentParser(description="tokenmill_amd: continuous-batching generation on one MI355X")
    add_engine_args(parser)
    parser.add_argument("--random", default=None, metavar="CONFIG",
                        help="a config.json (or its folder), or the name of a shipped shape (tiny-a, tiny-b, 0.5b, 7b, 32b): "
                             "run it with random weights instead of --model")
    parser.add_argument("--weights-seed", type=int, default=0, help="seed of the random weights")
    parser.add_argument("--prompt-ids", default=None, help='prompts as token ids: "1,2,3;4,5"')
    parser.add_argument("--prompt-lens", default=None, help="lengths of uniform-random prompts: 5,17,33")
    parser.add_argument("--prompt-seed", type=int, default=0)
    parser.add_argument("--max-tokens", type=int, default=256)
    parser.add_argument("--temperature", type=float, default=0.0)
    parser.add_argument("--top-k", type=int, default=-1)
    parser.add_argument("--top-p", type=float, default=1.0)
    parser.add_argument("--sample-seed", type=int, default=None,
                        help="seed of the sampling streams: prompt i uses seed + i (default: drawn from --seed)")
    parser.add_argument("--ignore-eos", action="store_true")
    parser.add_argument("--log-level", default="warning")
    args = parser.parse_args(argv)
    logging.basicConfig(level=args.log_level.upper(), format="%(asctime)s %(levelname)s %(name)s: %(message)s")
    if args.debug_steps:
        logging.getLogger("tokenmill_amd.engine").setLevel(logging.INFO)
    if bool(args.model) == bool(args.random):
        parser.error("give exactly one of --model DIR and --random CONFIG")
    if (args.prompt_ids is None) == (args.prompt_lens is None):
        parser.error("give exactly one of --prompt-ids and --prompt-lens")

    import torch

    from tokenmill_amd.engine.engine import LLMEngine
    from tokenmill_amd.sampling.sampler import SamplingParams

    cfg = engine_config_from_args(args)
    model = None
    if args.random:
        from tokenmill_amd.config.shapes import read_shape
        from tokenmill_amd.engine.loading import load_random_model, resolve_device, resolve_dtype

        config = read_shape(args.random)
        model = load_random_model(config, args.weights_seed, resolve_dtype(cfg.dtype), resolve_device(cfg.device),
                                  max_positions=cfg.max_model_len, pack_weights=cfg.pack_weights)
    engine = LLMEngine(cfg, model=model)
    if args.prompt_ids is not None:
        prompts = [[int(t) for t in part.split(",") if t.strip()] for part in args.prompt_ids.split(";") if part.strip()]
    else:
        g = torch.Generator().manual_seed(args.prompt_seed)
        vocab = engine.runner.vocab
        prompts = [torch.randint(0, vocab, (int(n),), generator=g).tolist() for n in args.prompt_lens.split(",")]
    # prompt i draws from the stream of seed + i (one seed for all would give every prompt the same draws);
    # without a seed the engine draws one per request from its own generator (--seed)
    params = [SamplingParams(max_tokens=args.max_tokens, temperature=args.temperature, top_k=args.top_k,
                             top_p=args.top_p, seed=None if args.sample_seed is None else args.sample_seed + i,
                             ignore_eos=args.ignore_eos) for i in range(len(prompts))]
    outputs = engine.generate(prompts, params)
    for i, (p, o) in enumerate(zip(prompts, outputs)):
        print(json.dumps({"prompt": i, "prompt_tokens": len(p), "output_ids": o}))
    return 0


if __name__ == "__main__":
    sys.exit(main())
