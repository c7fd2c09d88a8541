"""How many cache pages the engine makes: given, from a byte budget, or from the memory that is
left after the weights and the largest step (reference src/infer/engine/engine.py:44-84,
src/infer/engine/model_runner.py:99-118 size their pool the same three ways)."""
from __future__ import annotations

import torch

from tokenmill_amd.cache.manager import CacheManager
from tokenmill_amd.cache.pool import CachePools
from tokenmill_amd.config.engine_config import EngineConfig

GRAPH_SHAPES_RESERVED = 4       # captured steps of the largest size whose activations are kept out of the pool's budget


def largest_step_bytes(cfg: EngineConfig, model, dtype, device) -> tuple[int, int]:
    """Runs one step of ``max_num_batched_tokens`` tokens (prompts of at most ``max_model_len``) on a throw-away
    pool. Returns (bytes the allocator held at the peak, weights included; bytes of that peak that were the
    step's own activations)."""
    from tokenmill_amd.engine.runner import ModelRunner, StepEntry

    n = cfg.max_num_batched_tokens
    longest = min(n, cfg.max_model_len)
    lengths = [longest] * (n // longest) + ([n % longest] if n % longest else [])
    pages = sum(-(-s // cfg.block_size) for s in lengths)
    pools = CachePools(model, pages, cfg.block_size, len(lengths), dtype, device)
    manager = CacheManager(pools.windows, pages, cfg.block_size, len(lengths))
    runner = ModelRunner(model, pools, max_positions=cfg.max_model_len)
    torch.cuda.synchronize(device)
    before = torch.cuda.memory_allocated(device)          # weights and the throw-away pool
    pool_bytes = pools.nbytes
    torch.cuda.reset_peak_memory_stats(device)
    runner.step([StepEntry(manager.allocate(f"sizing-{i}", s), 0, [0] * s, [s - 1]) for i, s in enumerate(lengths)])
    torch.cuda.synchronize(device)
    peak = torch.cuda.max_memory_allocated(device)
    del runner, pools, manager
    torch.cuda.empty_cache()
    return max(peak - pool_bytes, 0), max(peak - before, 0)


def num_cache_pages(cfg: EngineConfig, model, dtype, device) -> int:
    """Pages per layer group: ``num_blocks`` as given; else ``kv_cache_mb``; else what
    ``gpu_memory_utilization`` of the card leaves after the weights, the largest step and, with
    ``hip_graphs``, the activations a few captured steps of that size keep. Never more than
    ``max_num_seqs`` requests of ``max_model_len`` tokens can use."""
    if cfg.num_blocks is not None:
        pages = cfg.num_blocks
    else:
        per_page = max(CachePools.bytes_per_token(model, dtype) * cfg.block_size, 1)
        if cfg.kv_cache_mb is not None:
            budget = int(cfg.kv_cache_mb * 2**20)
        else:
            peak, activations = largest_step_bytes(cfg, model, dtype, device)
            total = torch.cuda.get_device_properties(device).total_memory
            budget = int(total * cfg.gpu_memory_utilization) - peak
            if cfg.hip_graphs:
                budget -= GRAPH_SHAPES_RESERVED * activations
            if budget <= 0:
                raise RuntimeError("no memory left for the cache: lower --max-batched-tokens or raise "
                                   "--gpu-memory-utilization")
        pages = min(budget // per_page, cfg.max_num_seqs * (-(-cfg.max_model_len // cfg.block_size)))
    if pages < 2:
        raise RuntimeError("the cache budget gives fewer than two pages")
    return int(pages)
