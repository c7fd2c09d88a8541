"""y = x W^T + b with W stored [out, in] (reference src/infer/model/layers.py:139-140,159-160).

Several checkpoint tensors may be stacked along the output dimension into one matrix at load time
(q, k, v; gate, up), as the reference's loader does by row ranges
(reference src/infer/model/loader.py:44-46,68-70,111-116).
"""
from __future__ import annotations

import torch

from tokenmill_amd.hip import ops
from tokenmill_amd.parts.base import Part
from tokenmill_amd.weights.loader import TensorSpec


class Linear(Part):
    def __init__(self, in_features: int, out_features: list[int] | int, names: list[str] | str,
                 bias: bool = False, library_first: bool = False):
        self.in_features = in_features
        self.out_splits = [out_features] if isinstance(out_features, int) else list(out_features)
        self.names = [names] if isinstance(names, str) else list(names)
        assert len(self.names) == len(self.out_splits)
        self.out_features = sum(self.out_splits)
        self.has_bias = bias
        self.library_first = library_first              # a wide matrix the library reads fastest at any row count
        self.weight: torch.Tensor | None = None
        self.bias: torch.Tensor | None = None
        self.packed: ops.PackedWeight | None = None     # the matrix again in the order the decode kernels read
        self._desc = None                               # the matrix as the library's product rule takes it

    def tensor_specs(self, prefix: str) -> dict[str, TensorSpec]:
        specs = {}
        for name, n in zip(self.names, self.out_splits):
            specs[f"{prefix}{name}.weight"] = TensorSpec((n, self.in_features))
            if self.has_bias:
                specs[f"{prefix}{name}.bias"] = TensorSpec((n,))
        return specs

    def load(self, tensors, prefix: str) -> None:
        ws = [tensors[f"{prefix}{name}.weight"] for name in self.names]
        self.weight = ws[0] if len(ws) == 1 else torch.cat(ws, dim=0).contiguous()
        if self.has_bias:
            bs = [tensors[f"{prefix}{name}.bias"] for name in self.names]
            self.bias = bs[0] if len(bs) == 1 else torch.cat(bs, dim=0).contiguous()
            if self.weight.dtype == torch.float32 and self.bias.dtype != torch.float32:
                self.bias = self.bias.float()          # a 32-bit product adds a 32-bit bias
        self._desc = None

    def pack(self, rows, parts: list[int] | None = None) -> None:
        """Keep a second copy of a bfloat16 matrix in strip order (``ops.pack_weight``) for the products of
        decode steps, which read it about 15% faster that way; prompt-sized products keep reading the
        row-major one. ``rows``: rows of a strip, or a function that gives them (asked only if the matrix
        is packed). A matrix of another type or not on a GPU is left as it is."""
        w = self.weight
        if w is not None and w.dtype == torch.bfloat16 and w.is_cuda:
            self.packed = ops.pack_weight(w, rows() if callable(rows) else rows, parts)
            self._desc = None

    def describe(self):
        """The matrix, its packed copy and its bias as the kernel library takes them (kept until the tensors
        change); None while there is nothing on a GPU to describe."""
        if self._desc is None and self.weight is not None and self.weight.is_cuda and self.weight.is_contiguous() \
                and self.weight.dtype in (torch.float32, torch.bfloat16):
            self._desc = ops.linear_desc(self.weight, self.packed, self.bias, self.library_first)
        return self._desc

    def cost(self, rows: int, in_bytes: int | None = None, out_bytes: int | None = None) -> tuple[int, int]:
        """(bytes, flops) the product has to move and do for ``rows`` rows: the matrix once, the input and
        the output (``in_bytes`` / ``out_bytes`` per element, default the matrix's element size)."""
        e = self.weight.element_size()
        n, k = self.out_features, self.in_features
        moved = n * k * e + rows * k * (e if in_bytes is None else in_bytes) + rows * n * (e if out_bytes is None else out_bytes)
        if self.bias is not None:
            moved += self.bias.numel() * self.bias.element_size()
        return moved, 2 * rows * n * k

    def use_weight(self, weight: torch.Tensor) -> None:
        """Share another part's matrix (a tied output head)."""
        self.weight = weight
        self._desc = None

    def forward(self, x: torch.Tensor, out_dtype: torch.dtype | None = None,
                accumulate_into: torch.Tensor | None = None) -> torch.Tensor | None:
        """x [M, in] (row-strided views allowed) -> [M, out] in ``out_dtype`` (default: x's type).
        With ``accumulate_into`` (float32 [M, out]) the result may be added there by the product's own
        epilogue; then None is returned. Which kernel runs is the library's choice (``ops.linear``)."""
        w = self.weight
        out_dtype = out_dtype or x.dtype
        desc = self.describe()
        if accumulate_into is not None and w.dtype == x.dtype and ops.linear_accumulates(desc, x):
            ops.linear(desc, x, None, accum=accumulate_into)
            return None
        if w.dtype != x.dtype:
            # a matrix the checkpoint stores in 32-bit stays 32-bit: widen the activations for it
            x = ops.convert(x.contiguous(), torch.empty(x.shape, dtype=w.dtype, device=x.device))
        inner_dtype = torch.float32 if x.dtype == torch.float32 else out_dtype
        out = torch.empty((x.shape[0], self.out_features), dtype=inner_dtype, device=x.device)
        if x.shape[0]:
            ops.linear(desc, x, out)
        if out.dtype != out_dtype:
            out = ops.convert(out, torch.empty(out.shape, dtype=out_dtype, device=out.device))
        return out
