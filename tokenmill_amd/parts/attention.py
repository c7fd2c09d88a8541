"""Grouped-query attention over the paged cache (reference src/infer/model/layers.py:127-150,
src/infer/kv/context.py:63-80).

One fused q|k|v projection, position encoding and cache write in one kernel, then attention of
every token of the step over its own request's cache, then the output projection. Portions of
prompts and single decoded tokens go through the same call; the kernels read keys and values in
place through the block tables.
"""
from __future__ import annotations

import torch

from tokenmill_amd import profiling
from tokenmill_amd.hip import attention as attn_kernels
from tokenmill_amd.hip import gemm, ops
from tokenmill_amd.parts.base import (KVCacheSpec, KVCacheView, Mixer, NormedInput, PositionEncoding, StepContext,
                                      as_tensor)
from tokenmill_amd.parts.linear import Linear


MAX_HEAD_DIM = 256      # the widest head the generic attention kernel takes (the matrix-unit kernels: 32, 64, 96, 128)


class GQAttention(Mixer):
    def __init__(self, hidden: int, num_heads: int, num_kv_heads: int, head_dim: int, scale: float,
                 position: PositionEncoding, qkv_bias: bool = True, o_bias: bool = False,
                 window: int | None = None,
                 names: tuple[str, str, str, str] = ("q_proj", "k_proj", "v_proj", "o_proj")):
        if num_heads % num_kv_heads:
            raise ValueError(f"{num_heads} query heads do not divide into {num_kv_heads} kv heads")
        if head_dim % 4 or not 0 < head_dim <= MAX_HEAD_DIM:
            # said where the model is built, not by the first step that reaches a kernel
            raise ValueError(f"head size {head_dim}: the attention kernels take multiples of 4 up to {MAX_HEAD_DIM}")
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

    def prepare(self, pack_weights: bool) -> None:
        if not pack_weights:
            return
        if self.head_dim % 32 == 0:
            self.qkv.pack(lambda: ops.fused_qkv_strip_rows(self.num_heads, self.num_kv_heads, self.head_dim, self.hidden))
        self.o.pack(lambda: ops.skinny_strip_rows(self.hidden, self.q_size))

    def cache_spec(self):
        return KVCacheSpec(self.num_kv_heads, self.head_dim, self.window)

    def _fused_qkv(self, x, step: StepContext, cache: KVCacheView) -> torch.Tensor | None:
        """q [T, H*D] with k and v already in the cache, by the kernel that starts at the norm; None if
        that kernel does not take this step."""
        if not isinstance(x, NormedInput) or x.dtype != torch.bfloat16 or self.head_dim % 32:
            return None
        rms = x.fusable_rms()
        tables = getattr(self.position, "fusable_tables", lambda: None)()
        page = cache.k.shape[1]
        bias = self.qkv.bias
        if (rms is None or tables is None or not gemm.fused_decode_ok(x.resid, self.qkv.packed) or page & (page - 1)
                or step.max_context_len > self.position.max_positions
                or (bias is not None and bias.data_ptr() % 16)):
            return None
        q = torch.empty((x.num_tokens, self.q_size), dtype=torch.bfloat16, device=x.resid.device)
        write = cache.write
        ops.fused_norm_qkv_rope(x.resid, rms[0], rms[1], self.qkv.packed, self.qkv.bias, q, self.num_heads,
                                self.num_kv_heads, self.head_dim, tables[0], tables[1], step.positions,
                                step.groups[cache.group].slot_mapping if write else None,
                                cache.k if write else None, cache.v if write else None)
        return q

    def _panel_qkv(self, x: torch.Tensor, step: StepContext, cache: KVCacheView) -> torch.Tensor | None:
        """The same for 17 to 64 tokens, from the normed input; None if that kernel does not take this step."""
        tables = getattr(self.position, "fusable_tables", lambda: None)()
        page = cache.k.shape[1]
        bias = self.qkv.bias
        if (tables is None or self.head_dim % 32 or not gemm.panel_ok(x, self.qkv.packed) or page & (page - 1)
                or step.max_context_len > self.position.max_positions
                or (bias is not None and bias.data_ptr() % 16)):
            return None
        q = torch.empty((x.shape[0], self.q_size), dtype=torch.bfloat16, device=x.device)
        write = cache.write
        ops.panel_qkv_rope(x, self.qkv.packed, bias, q, self.num_heads, self.num_kv_heads, self.head_dim, tables[0],
                           tables[1], step.positions, step.groups[cache.group].slot_mapping if write else None,
                           cache.k if write else None, cache.v if write else None)
        return q

    def _attention_cost(self, step: StepContext, elem: int) -> tuple[int, int]:
        """Every key and value of the step's requests read once, q read and the output written; two
        products of 2 * head_dim flops per (query, visible key, head)."""
        keys_read = pairs = 0
        for start, n in zip(step.start_positions, step.q_lens):
            keys_read += min(start + n, self.window + n - 1) if self.window else start + n
            for i in range(n):
                pairs += min(start + i + 1, self.window) if self.window else start + i + 1
        moved = 2 * keys_read * self.kv_size * elem + 2 * step.num_tokens * self.q_size * elem
        return moved, 4 * pairs * self.num_heads * self.head_dim

    def forward(self, x, step: StepContext, cache: KVCacheView, residual: torch.Tensor | None = None):
        with profiling.label("qkv", lambda: self.qkv.cost(step.num_tokens)):       # with norm, rotary and cache write where fused
            q = self._fused_qkv(x, step, cache)
            if q is None:
                x = as_tensor(x)
                q = self._panel_qkv(x, step, cache)
            if q is None:
                q = self.qkv.forward(x)                                    # [T, (H + 2 KVH) D], q first
                self.position.encode_and_store(q, self.num_heads, self.num_kv_heads, self.head_dim, step, cache)
        out = torch.empty((q.shape[0], self.q_size), dtype=q.dtype, device=q.device)
        with profiling.label("attention", lambda: self._attention_cost(step, q.element_size())):
            attn_kernels.paged_attention(q, out, cache, step, self.num_heads, self.num_kv_heads, self.head_dim,
                                         self.scale, self.window or 0)
        with profiling.label("o_proj", lambda: self.o.cost(step.num_tokens)):
            return self.o.forward(out, accumulate_into=residual)
