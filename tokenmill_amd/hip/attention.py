"""Which attention kernels a step runs.

The step's entries are ordered with the single-token entries last. In bfloat16 those go to the
split-context MFMA decode kernel when it takes the head size, group and page size; everything
else (prompt portions, the true 32-bit path, unusual shapes) goes to the generic kernel.
"""
from __future__ import annotations

import torch

from tokenmill_amd.hip import ops
from tokenmill_amd.parts.base import KVCacheView, StepContext


def paged_attention(qkv: torch.Tensor, out: torch.Tensor, cache: KVCacheView, step: StepContext, H: int, KVH: int,
                    D: int, scale: float, window: int) -> torch.Tensor:
    """q = the first H*D columns of qkv; keys and values come from the cache (this step's included)."""
    g = step.groups[cache.group]
    T, S, nd = step.num_tokens, step.num_seqs, step.num_decode
    page = cache.k.shape[1]
    if nd and ops.attn_decode_mfma_supported(qkv.dtype, H, KVH, D, page):
        tp = T - nd
        if tp:
            ops.attn_paged_generic(qkv[:tp], out[:tp], cache.k, cache.v, g.block_tables, step.seq_of_token[:tp],
                                   step.positions[:tp], H, KVH, D, scale, window)
        ops.attn_decode_mfma(qkv[tp:], out[tp:], cache.k, cache.v, g.block_tables[S - nd:], step.context_lens[S - nd:],
                             H, KVH, D, scale, window, step.max_decode_context)
        return out
    return ops.attn_paged_generic(qkv, out, cache.k, cache.v, g.block_tables, step.seq_of_token, step.positions,
                                  H, KVH, D, scale, window)
