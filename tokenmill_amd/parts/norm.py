"""RMSNorm fused with the residual add (reference src/infer/model/layers.py:35-44,
src/infer/model/qwen2.py:22-23)."""
from __future__ import annotations

import torch

from tokenmill_amd import profiling
from tokenmill_amd.hip import ops
from tokenmill_amd.parts.base import Norm
from tokenmill_amd.weights.loader import TensorSpec


class RMSNorm(Norm):
    """out = weight * round(x * rsqrt(mean(x^2) + eps)); the weight is used as it is (not 1 + w)."""

    def __init__(self, hidden: int, eps: float):
        self.hidden = hidden
        self.eps = float(eps)
        self.weight: torch.Tensor | None = None

    def tensor_specs(self, prefix: str):
        return {f"{prefix}weight": TensorSpec((self.hidden,), init="ones")}

    def load(self, tensors, prefix: str) -> None:
        self.weight = tensors[f"{prefix}weight"]

    def add_norm(self, resid, delta, out_dtype, rows=None):
        n = resid.shape[0] if rows is None else rows.numel()
        out = torch.empty((n, self.hidden), dtype=out_dtype, device=resid.device)
        with profiling.label("norm", lambda: (n * self.hidden * (4 + (0 if rows is not None else 4) + out.element_size()
                                                                 + (out.element_size() if delta is not None else 0)), 0)):
            return ops.add_rmsnorm(resid, delta, self.weight, self.eps, out, rows)

    def rms_params(self):
        return self.weight, self.eps
