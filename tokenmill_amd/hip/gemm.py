"""Which matrix-product kernel a Linear runs.

float32: the LDS-tiled kernel with 32-bit multiply-adds (a true 32-bit product, fixed summation
order). bfloat16: up to 64 rows the MFMA kernel that streams the matrix once (decode steps); more
rows go to the library's matrix product, as the reference's engine does for all of its products
(reference src/infer/model/layers.py:144,150,163-164); shapes neither takes run the tiled kernel.
"""
from __future__ import annotations

import torch

from tokenmill_amd.hip import ops

SKINNY_ROWS = 64


def _skinny_ok(x: torch.Tensor, w: torch.Tensor) -> bool:
    K = x.shape[1]
    stride = x.stride(0) if x.shape[0] > 1 else K
    return (x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and K % 8 == 0 and stride % 8 == 0
            and x.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0)


def linear(x: torch.Tensor, w: torch.Tensor, bias: torch.Tensor | None, out: torch.Tensor) -> torch.Tensor:
    """out[M, N] = x[M, K] @ w[N, K]^T (+ bias)."""
    M = x.shape[0]
    if M == 0:
        return out
    if x.dtype != torch.bfloat16:
        return ops.gemm_nt_tiled(x, w, bias, out)
    skinny = _skinny_ok(x, w)
    if skinny and M <= SKINNY_ROWS:
        return ops.gemm_skinny(x, w, bias, out)
    if out.dtype == torch.bfloat16 and (bias is None or bias.dtype == torch.bfloat16) and out.is_contiguous():
        if bias is None:
            torch.mm(x, w.t(), out=out)
        else:
            torch.addmm(bias, x, w.t(), out=out)
        return out
    if skinny:                                   # 32-bit results for many rows (logits of a replay)
        for r0 in range(0, M, SKINNY_ROWS):
            ops.gemm_skinny(x[r0:r0 + SKINNY_ROWS], w, bias, out[r0:r0 + SKINNY_ROWS])
        return out
    return ops.gemm_nt_tiled(x, w, bias, out)


def gate_up_silu(x: torch.Tensor, w_gate_up: torch.Tensor, out: torch.Tensor) -> bool:
    """out[M, I] = silu(x Wg^T) * (x Wu^T) in one kernel, if a fused kernel takes this shape."""
    if x.shape[0] <= SKINNY_ROWS and _skinny_ok(x, w_gate_up):
        ops.gemm_skinny(x, w_gate_up, None, out, silu=True)
        return True
    return False


def linear_accumulate(x: torch.Tensor, w: torch.Tensor, bias: torch.Tensor | None, accum: torch.Tensor) -> bool:
    """accum[M, N] (float32) += round_bf16(x @ w^T + bias) in the product's epilogue, if a kernel does that
    for this shape."""
    if 0 < x.shape[0] <= SKINNY_ROWS and _skinny_ok(x, w):
        ops.gemm_skinny(x, w, bias, None, accum=accum)
        return True
    return False


def fused_decode_ok(resid: torch.Tensor, w: torch.Tensor) -> bool:
    """Can the norm-fused decode products take this residual and matrix?"""
    M, K = resid.shape
    return (0 < M <= ops.FUSED_DECODE_ROWS and w.dtype == torch.bfloat16 and K % 8 == 0 and ops.fused_lds_fits(K)
            and resid.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0)
