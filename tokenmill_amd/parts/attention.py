"""Grouped-query attention over the paged cache (reference src/infer/model/layers.py:127-150,
src/infer/kv/context.py:63-80).

One fused q|k|v projection, position encoding and cache write in one kernel, then attention of
every token of the step over its own request's cache, then the output projection. Portions of
prompts and single decoded tokens go through the same call; the kernels read keys and values in
place through the block tables.
"""
from __future__ import annotations

import torch

from tokenmill_amd.hip import attention as attn_kernels
from tokenmill_amd.parts.base import KVCacheSpec, KVCacheView, Mixer, PositionEncoding, StepContext
from tokenmill_amd.parts.linear import Linear


class GQAttention(Mixer):
    def __init__(self, hidden: int, num_heads: int, num_kv_heads: int, head_dim: int, scale: float,
                 position: PositionEncoding, qkv_bias: bool = True, o_bias: bool = False,
                 window: int | None = None,
                 names: tuple[str, str, str, str] = ("q_proj", "k_proj", "v_proj", "o_proj")):
        if num_heads % num_kv_heads:
            raise ValueError(f"{num_heads} query heads do not divide into {num_kv_heads} kv heads")
        self.hidden, self.num_heads, self.num_kv_heads, self.head_dim = hidden, num_heads, num_kv_heads, head_dim
        self.scale = float(scale)
        self.window = window
        self.position = position
        q, kv = num_heads * head_dim, num_kv_heads * head_dim
        self.q_size, self.kv_size = q, kv
        self.qkv = Linear(hidden, [q, kv, kv], list(names[:3]), bias=qkv_bias)
        self.o = Linear(q, hidden, names[3], bias=o_bias)

    def tensor_specs(self, prefix: str):
        return {**self.qkv.tensor_specs(prefix), **self.o.tensor_specs(prefix), **self.position.tensor_specs(prefix)}

    def load(self, tensors, prefix: str) -> None:
        self.qkv.load(tensors, prefix)
        self.o.load(tensors, prefix)
        self.position.load(tensors, prefix)

    def cache_spec(self):
        return KVCacheSpec(self.num_kv_heads, self.head_dim, self.window)

    def forward(self, x: torch.Tensor, step: StepContext, cache: KVCacheView) -> torch.Tensor:
        qkv = self.qkv.forward(x)                                          # [T, (H + 2 KVH) D]
        self.position.encode_and_store(qkv, self.num_heads, self.num_kv_heads, self.head_dim, step, cache)
        out = torch.empty((x.shape[0], self.q_size), dtype=qkv.dtype, device=x.device)
        attn_kernels.paged_attention(qkv, out, cache, step, self.num_heads, self.num_kv_heads, self.head_dim,
                                     self.scale, self.window or 0)
        return self.o.forward(out)
