"""Which matrix-product kernel a Linear runs.

float32: the LDS-tiled kernel with 32-bit multiply-adds (a true 32-bit product, fixed summation
order). bfloat16: MFMA kernels of this library where one fits the shape; the tiled kernel
otherwise.
"""
from __future__ import annotations

import torch

from tokenmill_amd.hip import ops


def linear(x: torch.Tensor, w: torch.Tensor, bias: torch.Tensor | None, out: torch.Tensor) -> torch.Tensor:
    return ops.gemm_nt_tiled(x, w, bias, out)
