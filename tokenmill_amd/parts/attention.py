"""Grouped-query attention over the paged cache (reference src/infer/model/layers.py:127-150,
src/infer/kv/context.py:63-80).

One fused q|k|v projection, position encoding and cache write, then attention of every token of the
step over its own request's cache, then the output projection. Portions of prompts and single decoded
tokens go through the same call; the kernels read keys and values in place through the block tables.
The part describes all of that to the kernel library as one operation (``emit``); which kernels run
for a step is decided there.
"""
from __future__ import annotations

import torch

from tokenmill_amd import profiling
from tokenmill_amd.hip import ops
from tokenmill_amd.hip.program import StepProgram
from tokenmill_amd.parts.base import (KVCacheSpec, KVCacheView, Mixer, Norm, NormedInput, PositionEncoding, StepContext,
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
        self._own: dict = {}                    # one-operation programs for calls of ``forward``

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

    # --- the operation ------------------------------------------------------------------------------------

    def emit(self, program, norm: Norm | None, cache, encoded_outside: bool = False) -> int | None:
        """``encoded_outside``: the operation will only ever be handed q|k|v that are already encoded and stored
        (the way a position encoding the library does not know is run)."""
        rotation = () if encoded_outside else self.position.rotation()
        if rotation is None or not isinstance(cache, KVCacheView):
            return None
        return program.attention(self, norm, self.qkv, self.o, rotation, cache, self.num_heads, self.num_kv_heads,
                                 self.head_dim, self.scale, self.window)

    def cost(self, label: str, step: StepContext | None, rows: int) -> tuple[int, int]:
        if label == "qkv":
            return self.qkv.cost(rows)                  # with norm, rotary and cache write where fused
        if label == "o_proj":
            return self.o.cost(rows)
        # attention: every key and value of the step's requests read once, q read and the output written; two
        # products of 2 * head_dim flops per (query, visible key, head)
        elem = self.qkv.weight.element_size()
        keys_read = pairs = 0
        for start, n in zip(step.start_positions, step.q_lens):
            keys_read += min(start + n, self.window + n - 1) if self.window else start + n
            if self.window:
                pairs += sum(min(start + i + 1, self.window) for i in range(n))
            else:
                pairs += n * start + n * (n + 1) // 2
        moved = 2 * keys_read * self.kv_size * elem + 2 * step.num_tokens * self.q_size * elem
        return moved, 4 * pairs * self.num_heads * self.head_dim

    def _alone(self, norm: Norm | None, cache: KVCacheView, dtype, encoded_outside: bool = False):
        """This mixer's operation as a program of its own, for calls of ``forward``."""
        key = (id(norm), id(cache.k), cache.write, dtype, encoded_outside)
        entry = self._own.get(key)
        if entry is None:
            program = StepProgram(dtype, self.hidden, cache.k.device)
            op = self.emit(program, norm, cache, encoded_outside)
            if op is None:
                raise ops.KernelArgumentError("the kernel library has no attention operation for these tensors")
            entry = self._own[key] = (program, op, norm, cache)
        return entry[0], entry[1]

    def forward(self, x, step: StepContext, cache: KVCacheView, residual: torch.Tensor | None = None):
        """The same operation called by itself: by a block that is not described to a step program, or a test."""
        if self.position.rotation() is None:
            # an encoding the library does not know: project, let it encode and store, attend from there
            x = as_tensor(x)
            with profiling.label("qkv", lambda: self.qkv.cost(x.shape[0])):
                qkv = self.qkv.forward(x)
                self.position.encode_and_store(qkv, self.num_heads, self.num_kv_heads, self.head_dim, step, cache)
            program, op = self._alone(None, cache, x.dtype, encoded_outside=True)
            return program.run_one(op, step, resid=residual, qkv=qkv, accumulate=residual is not None)
        if isinstance(x, NormedInput) and x.lazy:
            program, op = self._alone(x.norm, cache, x.dtype)
            resid, delta = x.take()
            return program.run_one(op, step, resid=resid, delta=delta, accumulate=residual is resid)
        x = as_tensor(x)
        program, op = self._alone(None, cache, x.dtype)
        return program.run_one(op, step, resid=residual, x=x.contiguous(), accumulate=residual is not None)
