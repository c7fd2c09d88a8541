"""Which matrix-product kernel a Linear runs.

float32: up to 16 rows a matrix-vector kernel with 32-bit multiply-adds that streams the matrix once;
beyond that the kernel on the 32-bit matrix unit (32-bit products and sums, a fixed summation order),
or for shapes it does not take the LDS-tiled kernel on the vector unit (the same guarantees).
bfloat16: up to 16 rows (decode steps) the MFMA kernels of this library that stream the matrix once
(from its packed copy where the Linear keeps one) and carry the layer's epilogue (bias, rotary +
cache write, SiLU·up, residual add) or start at the norm; from 17 to 48 rows the q|k|v and gate|up
products keep the normed input in LDS and carry the same epilogues; everything else goes to the
library's matrix product (hipBLASLt, called from this package's own library with the plan of every
shape kept), as the reference's engine uses a library for all of its products (reference
src/infer/model/layers.py:144,150,163-164, src/infer/model/qwen2.py:51-52); measured on an MI355X
the library is the faster one from about 32 rows on for a plain product, and for the wide output
head at any row count. Shapes neither takes run the tiled kernel.
"""
from __future__ import annotations

import torch

from tokenmill_amd.hip import ops

SKINNY_ROWS = 16            # most rows the skinny kernels are preferred for
PANEL_ROWS = 48             # most rows the products that keep the normed input in LDS are preferred for (they
                            # take 64; measured, the library and the element-wise kernels are as fast from 56 on)
SKINNY_MAX_ROWS = 64        # most rows they can take


def _skinny_ok(x: torch.Tensor, w: torch.Tensor) -> bool:
    K = x.shape[1]
    stride = x.stride(0) if x.shape[0] > 1 else K
    return (x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and K % 8 == 0 and stride % 8 == 0
            and x.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0)


def linear(x: torch.Tensor, w: torch.Tensor, bias: torch.Tensor | None, out: torch.Tensor, packed=None,
           library_first: bool = False) -> torch.Tensor:
    """out[M, N] = x[M, K] @ w[N, K]^T (+ bias). ``packed``: w in strip order, read instead where it serves.
    ``library_first``: the owner of w asks for the library's product at any row count (an output head)."""
    M = x.shape[0]
    if M == 0:
        return out
    if packed is not None and len(packed.parts) == 1 and out.stride(1) == 1 and _packed_ok(x, packed) \
            and not library_first:
        return ops.gemm_skinny(x, packed, bias, out)
    if x.dtype != torch.bfloat16:
        if ops.gemv_f32_ok(x, w, bias, out):                    # a decode step of the 32-bit path
            return ops.gemv_f32(x, w, bias, out)
        if ops.gemm_f32_mfma_ok(x, w, bias, out):               # a prompt-sized step of it: the 32-bit matrix unit
            return ops.gemm_f32_mfma(x, w, bias, out)
        return ops.gemm_nt_tiled(x, w, bias, out)
    skinny = _skinny_ok(x, w)
    library = w.dtype == torch.bfloat16 and x.stride(1) == 1 and out.stride(1) == 1
    if library and library_first and ops.gemm_library(x, w, bias, out):
        return out
    if skinny and M <= SKINNY_ROWS:
        return ops.gemm_skinny(x, w, bias, out)
    if library and ops.gemm_library(x, w, bias, out):
        return out
    if skinny:                                   # 32-bit results for many rows, 64 rows a call
        for r0 in range(0, M, SKINNY_MAX_ROWS):
            ops.gemm_skinny(x[r0:r0 + SKINNY_MAX_ROWS], w, bias, out[r0:r0 + SKINNY_MAX_ROWS])
        return out
    return ops.gemm_nt_tiled(x, w, bias, out)


def _packed_ok(x: torch.Tensor, packed) -> bool:
    K = x.shape[1]
    stride = x.stride(0) if x.shape[0] > 1 else K
    return (packed is not None and 0 < x.shape[0] <= ops.PACKED_ROWS and x.dtype == torch.bfloat16 and K == packed.k
            and K % 8 == 0 and stride % 8 == 0 and x.stride(1) == 1 and x.data_ptr() % 16 == 0)


def gate_up_silu(x: torch.Tensor, w_gate_up: torch.Tensor, out: torch.Tensor, packed=None) -> bool:
    """out[M, I] = silu(x Wg^T) * (x Wu^T) in one kernel, if a fused kernel takes this shape. ``packed``:
    the same matrix in strip order, read instead where it serves."""
    if _packed_ok(x, packed) and packed.rows == 16 and len(packed.parts) == 2:
        ops.gemm_skinny(x, packed, None, out, silu=True)
        return True
    if x.shape[0] <= SKINNY_ROWS and _skinny_ok(x, w_gate_up):
        ops.gemm_skinny(x, w_gate_up, None, out, silu=True)
        return True
    if panel_ok(x, packed) and packed.rows == 16 and len(packed.parts) == 2 and out.shape[1] % 4 == 0:
        ops.panel_gate_up_silu(x, packed, out)
        return True
    return False


def panel_ok(x: torch.Tensor, packed) -> bool:
    """Can the products that keep the normed input in LDS (17 to 64 tokens) take x and this packed matrix?"""
    if packed is None or x.dim() != 2:
        return False
    M, K = x.shape
    stride = x.stride(0) if M > 1 else K
    return (ops.PACKED_ROWS < M <= PANEL_ROWS and x.dtype == torch.bfloat16 and K == packed.k and x.stride(1) == 1
            and stride % 8 == 0 and x.data_ptr() % 16 == 0 and ops.panel_fits(M, K))


def linear_accumulate(x: torch.Tensor, w: torch.Tensor, bias: torch.Tensor | None, accum: torch.Tensor,
                      packed=None) -> bool:
    """accum[M, N] (float32) += round_bf16(x @ w^T + bias) in the product's epilogue, if a kernel does that
    for this shape. ``packed``: the same matrix in strip order, read instead where it serves."""
    if _packed_ok(x, packed) and len(packed.parts) == 1:
        ops.gemm_skinny(x, packed, bias, None, accum=accum)
        return True
    if 0 < x.shape[0] <= SKINNY_ROWS and _skinny_ok(x, w):
        ops.gemm_skinny(x, w, bias, None, accum=accum)
        return True
    return False


def fused_decode_ok(resid: torch.Tensor, packed) -> bool:
    """Can the norm-fused decode products take this residual and (packed) matrix?"""
    M, K = resid.shape
    return (packed is not None and 0 < M <= ops.FUSED_DECODE_ROWS and K == packed.k and K % 8 == 0
            and ops.fused_lds_fits(M, K) and resid.data_ptr() % 16 == 0)
