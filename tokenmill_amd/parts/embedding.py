"""Token embedding and output head (reference src/infer/model/qwen2.py:30-33,39-52)."""
from __future__ import annotations

import torch

from tokenmill_amd import profiling
from tokenmill_amd.hip import ops
from tokenmill_amd.parts.base import Part
from tokenmill_amd.parts.linear import Linear
from tokenmill_amd.weights.loader import TensorSpec


class TokenEmbedding(Part):
    """x = E[ids], no scaling; rows are widened into the 32-bit residual stream."""

    def __init__(self, vocab: int, hidden: int, name: str = "weight"):
        self.vocab, self.hidden, self.name = vocab, hidden, name
        self.weight: torch.Tensor | None = None

    def tensor_specs(self, prefix: str):
        return {f"{prefix}{self.name}": TensorSpec((self.vocab, self.hidden))}

    def load(self, tensors, prefix: str) -> None:
        self.weight = tensors[f"{prefix}{self.name}"]

    def emit(self, program) -> int | None:
        return program.embedding(self, self.weight)

    def cost(self, label, step, rows):
        return rows * self.hidden * (self.weight.element_size() + 4), 0

    def forward(self, token_ids: torch.Tensor) -> torch.Tensor:
        out = torch.empty((token_ids.numel(), self.hidden), dtype=torch.float32, device=token_ids.device)
        with profiling.label("embed", lambda: self.cost("embed", None, token_ids.numel())):
            return ops.embed_gather(self.weight, token_ids, out)


class OutputHead(Part):
    """logits = h W^T in 32-bit, W the embedding table itself when tied (no second copy)."""

    def __init__(self, hidden: int, vocab: int, tied_to: TokenEmbedding | None, name: str = "lm_head"):
        self.hidden, self.vocab, self.tied_to = hidden, vocab, tied_to
        self.proj = Linear(hidden, vocab, name, bias=False, library_first=True)

    def tensor_specs(self, prefix: str):
        return {} if self.tied_to is not None else self.proj.tensor_specs(prefix)

    def load(self, tensors, prefix: str) -> None:
        if self.tied_to is not None:
            self.proj.use_weight(self.tied_to.weight)
        else:
            self.proj.load(tensors, prefix)

    def emit(self, program, norm) -> int | None:
        """logits = proj(norm(resid[logit rows])): the final norm and this head as one operation."""
        return program.head(self, norm, self.proj, self.vocab)

    def cost(self, label, step, rows):
        n = step.num_logit_rows if step is not None else rows
        if label == "norm":
            e = self.proj.weight.element_size()
            return n * self.hidden * (4 + e), 0
        return self.proj.cost(n, out_bytes=4)

    def forward(self, h: torch.Tensor) -> torch.Tensor:
        with profiling.label("head", lambda: self.proj.cost(h.shape[0], out_bytes=4)):
            return self.proj.forward(h, out_dtype=torch.float32)
