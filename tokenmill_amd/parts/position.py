"""Position encodings applied to q and k before they are cached.

RotaryEmbedding: reference src/infer/model/layers.py:47-64. The cos/sin table is built once on
the host in 32-bit with the reference's expression and uploaded; the rotation runs in 32-bit in
the kernel that also stores k and v into the cache.
"""
from __future__ import annotations

import torch

from tokenmill_amd.hip import ops
from tokenmill_amd.parts.base import KVCacheView, PositionEncoding, StepContext


class RotaryEmbedding(PositionEncoding):
    """Pairs (j, j + rotary_dim/2) of each head rotate by position * theta^(-2j/rotary_dim)."""

    def __init__(self, head_dim: int, theta: float, max_positions: int, rotary_dim: int | None = None):
        self.head_dim = head_dim
        self.rotary_dim = rotary_dim or head_dim
        if self.rotary_dim % 2 or self.rotary_dim > head_dim:
            raise ValueError(f"rotary_dim {self.rotary_dim} must be even and at most head_dim {head_dim}")
        self.theta = float(theta)
        self.max_positions = max_positions
        self.cos: torch.Tensor | None = None
        self.sin: torch.Tensor | None = None

    def build_tables(self, device) -> None:
        d = self.rotary_dim
        inv_freq = 1.0 / (self.theta ** (torch.arange(0, d, 2, dtype=torch.int64).float() / d))
        freqs = torch.outer(torch.arange(self.max_positions).float(), inv_freq)     # [max_pos, d/2]
        self.cos = freqs.cos().contiguous().to(device)
        self.sin = freqs.sin().contiguous().to(device)

    def load(self, tensors, prefix: str) -> None:
        device = next(iter(tensors.values())).device
        if self.cos is None or self.cos.device != device:
            self.build_tables(device)

    def encode_and_store(self, qkv, num_heads, num_kv_heads, head_dim, step: StepContext, cache: KVCacheView | None):
        if step.max_context_len > self.max_positions:
            raise ValueError(f"position {step.max_context_len - 1} is beyond the rotary table "
                             f"({self.max_positions} positions)")
        write = cache is not None and cache.write
        ops.rope_kv_write(qkv, num_heads, num_kv_heads, head_dim, self.cos, self.sin, step.positions,
                          step.groups[cache.group].slot_mapping if write else None,
                          cache.k if write else None, cache.v if write else None)

    def rotation(self):
        """(cos, sin, rotary width, positions): what the kernel library's attention operation rotates by."""
        return (self.cos, self.sin, self.rotary_dim, self.max_positions) if self.cos is not None else None


class NoPositionEncoding(PositionEncoding):
    """Stores k and v; q and k stay as they are."""

    def rotation(self):
        return ()

    def encode_and_store(self, qkv, num_heads, num_kv_heads, head_dim, step: StepContext, cache: KVCacheView | None):
        if cache is not None and cache.write:
            ops.rope_kv_write(qkv, num_heads, num_kv_heads, head_dim, None, None, None,
                              step.groups[cache.group].slot_mapping, cache.k, cache.v)
