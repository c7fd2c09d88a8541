"""SwiGLU feed-forward: down(silu(gate(x)) * up(x)), gate and up stacked into one product
(reference src/infer/model/layers.py:153-164)."""
from __future__ import annotations

import torch

from tokenmill_amd.hip import ops
from tokenmill_amd.hip.program import StepProgram
from tokenmill_amd.parts.base import FeedForward, Norm, NormedInput, StepContext, as_tensor
from tokenmill_amd.parts.linear import Linear


class SwiGLU(FeedForward):
    def __init__(self, hidden: int, intermediate: int, bias: bool = False,
                 names: tuple[str, str, str] = ("gate_proj", "up_proj", "down_proj")):
        self.hidden, self.intermediate = hidden, intermediate
        self.gate_up = Linear(hidden, [intermediate, intermediate], list(names[:2]), bias=bias)
        self.down = Linear(intermediate, hidden, names[2], bias=bias)
        self._own: dict = {}                    # one-operation programs for calls of ``forward``

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

    def emit(self, program, norm: Norm | None) -> int | None:
        if self.gate_up.bias is not None or self.down.bias is not None:
            return None                         # the library's operation has no biases
        return program.feed_forward(self, norm, self.gate_up, self.down, self.intermediate)

    def cost(self, label: str, step: StepContext | None, rows: int) -> tuple[int, int]:
        return self.gate_up.cost(rows) if label == "gate_up" else self.down.cost(rows)   # gate_up: with norm and SiLU*up

    def _alone(self, norm: Norm | None, dtype, device):
        key = (id(norm), dtype)
        entry = self._own.get(key)
        if entry is None:
            program = StepProgram(dtype, self.hidden, device)
            op = self.emit(program, norm)
            entry = self._own[key] = (program, op, norm)
        return entry[0], entry[1]

    def forward(self, x, step: StepContext | None = None, residual: torch.Tensor | None = None):
        """The same operation called by itself: by a block or a feed-forward that is not described to a step
        program (an expert of a routed one), or a test."""
        if isinstance(x, NormedInput) and x.lazy:
            program, op = self._alone(x.norm, x.dtype, x.resid.device)
            if op is not None:
                resid, delta = x.take()
                return program.run_one(op, None, resid=resid, delta=delta, accumulate=residual is resid, rows=resid.shape[0])
        x = as_tensor(x)
        program, op = self._alone(None, x.dtype, x.device)
        if op is None:                          # with biases: the two products and the activation one by one
            act = torch.empty((x.shape[0], self.intermediate), dtype=x.dtype, device=x.device)
            ops.silu_mul(self.gate_up.forward(x), act)
            return self.down.forward(act, accumulate_into=residual)
        if x.shape[0] == 0:
            return None if residual is not None else torch.empty_like(x)
        return program.run_one(op, None, resid=residual, x=x.contiguous(), accumulate=residual is not None, rows=x.shape[0])
