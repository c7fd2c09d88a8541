"""Which attention kernels a step runs.

The step's entries are ordered with the single-token entries last. In bfloat16, when the head
size and page size allow, prompt portions go to the flash-style MFMA kernel and single tokens to
the split-context MFMA decode kernel. In float32 prompt portions go to the flash-style kernel on
the 32-bit MFMA. Everything else (single tokens in float32, unusual shapes) goes to the generic kernel.
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
    tp = T - nd
    page = cache.k.shape[1]
    # every kernel below walks a request's block table up to its newest position: the table must reach that far
    if step.max_context_len > g.block_tables.shape[1] * page:
        raise ops.KernelArgumentError(f"attention: a context of {step.max_context_len} positions and block tables of "
                                      f"{g.block_tables.shape[1]} pages of {page}")
    done_prefill = done_decode = False
    if tp and step.prefill_tiles is not None and ops.attn_prefill_mfma_supported(qkv.dtype, H, KVH, D, page):
        ops.attn_prefill_mfma(qkv, out, cache.k, cache.v, g.block_tables, step.prefill_tiles, H, KVH, D, scale, window)
        done_prefill = True
    elif tp and step.prefill_tiles is not None and ops.attn_prefill_f32_supported(qkv.dtype, H, KVH, D, page) \
            and qkv.stride(0) % 4 == 0 and qkv.data_ptr() % 16 == 0:
        ops.attn_prefill_f32(qkv, out, cache.k, cache.v, g.block_tables, step.prefill_tiles, H, KVH, D, scale, window)
        done_prefill = True
    if nd and ops.attn_decode_mfma_supported(qkv.dtype, H, KVH, D, page):
        ops.attn_decode_mfma(qkv[tp:], out[tp:], cache.k, cache.v, g.block_tables[S - nd:], step.context_lens[S - nd:],
                             H, KVH, D, scale, window, step.max_decode_context)
        done_decode = True
    if tp and not done_prefill and nd and not done_decode:
        return ops.attn_paged_generic(qkv, out, cache.k, cache.v, g.block_tables, step.seq_of_token, step.positions,
                                      H, KVH, D, scale, window)
    if tp and not done_prefill:
        ops.attn_paged_generic(qkv[:tp], out[:tp], cache.k, cache.v, g.block_tables, step.seq_of_token[:tp],
                               step.positions[:tp], H, KVH, D, scale, window)
    if nd and not done_decode:
        ops.attn_paged_generic(qkv[tp:], out[tp:], cache.k, cache.v, g.block_tables, step.seq_of_token[tp:],
                               step.positions[tp:], H, KVH, D, scale, window)
    return out
