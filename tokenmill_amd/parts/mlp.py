"""SwiGLU feed-forward: down(silu(gate(x)) * up(x)), gate and up stacked into one product
(reference src/infer/model/layers.py:153-164)."""
from __future__ import annotations

import torch

from tokenmill_amd import profiling
from tokenmill_amd.hip import gemm, ops
from tokenmill_amd.parts.base import FeedForward, NormedInput, StepContext, as_tensor
from tokenmill_amd.parts.linear import Linear


class SwiGLU(FeedForward):
    def __init__(self, hidden: int, intermediate: int, bias: bool = False,
                 names: tuple[str, str, str] = ("gate_proj", "up_proj", "down_proj")):
        self.hidden, self.intermediate = hidden, intermediate
        self.gate_up = Linear(hidden, [intermediate, intermediate], list(names[:2]), bias=bias)
        self.down = Linear(intermediate, hidden, names[2], bias=bias)

    def tensor_specs(self, prefix: str):
        return {**self.gate_up.tensor_specs(prefix), **self.down.tensor_specs(prefix)}

    def load(self, tensors, prefix: str) -> None:
        self.gate_up.load(tensors, prefix)
        self.down.load(tensors, prefix)

    def prepare(self, pack_weights: bool) -> None:
        if not pack_weights:
            return
        self.gate_up.pack(16, [self.intermediate, self.intermediate])
        self.down.pack(lambda: ops.skinny_strip_rows(self.hidden, self.intermediate))

    def forward(self, x, step: StepContext | None = None, residual: torch.Tensor | None = None):
        rows = x.num_tokens if isinstance(x, NormedInput) else x.shape[0]
        with profiling.label("gate_up", lambda: self.gate_up.cost(rows)):          # with norm and SiLU*up where fused
            act = self._activation(x)
        with profiling.label("down", lambda: self.down.cost(rows)):
            return self.down.forward(act, accumulate_into=residual)

    def _activation(self, x) -> torch.Tensor:
        """silu(gate(x)) * up(x), [T, intermediate]."""
        w = self.gate_up.weight
        act = None
        if isinstance(x, NormedInput) and x.dtype == torch.bfloat16 and self.gate_up.bias is None and \
                self.intermediate % 4 == 0:
            rms = x.fusable_rms()
            if rms is not None and gemm.fused_decode_ok(x.resid, self.gate_up.packed):   # the kernel that starts at the norm
                act = torch.empty((x.num_tokens, self.intermediate), dtype=torch.bfloat16, device=x.resid.device)
                ops.fused_norm_gate_up_silu(x.resid, rms[0], rms[1], self.gate_up.packed, act)
        if act is None:
            x = as_tensor(x)
            act = torch.empty((x.shape[0], self.intermediate), dtype=x.dtype, device=x.device)
            if not (w.dtype == x.dtype and self.gate_up.bias is None
                    and gemm.gate_up_silu(x, w, act, packed=self.gate_up.packed)):
                ops.silu_mul(self.gate_up.forward(x), act)
        return act
