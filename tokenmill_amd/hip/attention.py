"""Which attention kernel a step runs."""
from __future__ import annotations

import torch

from tokenmill_amd.hip import ops
from tokenmill_amd.parts.base import KVCacheView, StepContext


def paged_attention(qkv: torch.Tensor, out: torch.Tensor, cache: KVCacheView, step: StepContext, H: int, KVH: int,
                    D: int, scale: float, window: int) -> torch.Tensor:
    """q = the first H*D columns of qkv; keys and values come from the cache (this step's included)."""
    g = step.groups[cache.group]
    return ops.attn_paged_generic(qkv, out, cache.k, cache.v, g.block_tables, step.seq_of_token, step.positions,
                                  H, KVH, D, scale, window)
