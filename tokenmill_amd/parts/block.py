"""The arrangement of parts in a layer.

PreNormBlock: h = x + mixer(norm_in(x)); y = h + ffn(norm_post(h))
(reference src/infer/model/qwen2.py:13-23). The residual stream is a 32-bit tensor that the
block updates in place; each add is fused into the norm that follows it, so a block takes the
not-yet-added output of the previous block (``delta``) and returns its own.
"""
from __future__ import annotations

import torch

from tokenmill_amd.parts.base import FeedForward, Mixer, Norm, NormedInput, Part, StepContext


class PreNormBlock(Part):
    def __init__(self, norm_in: Norm, mixer: Mixer, norm_post: Norm, ffn: FeedForward,
                 names: tuple[str, str, str, str] = ("input_layernorm.", "self_attn.",
                                                     "post_attention_layernorm.", "mlp.")):
        self.norm_in, self.mixer, self.norm_post, self.ffn = norm_in, mixer, norm_post, ffn
        self.names = names

    def _parts(self):
        return zip((self.norm_in, self.mixer, self.norm_post, self.ffn), self.names)

    def tensor_specs(self, prefix: str):
        specs = {}
        for part, name in self._parts():
            specs.update(part.tensor_specs(prefix + name))
        return specs

    def load(self, tensors, prefix: str) -> None:
        for part, name in self._parts():
            part.load(tensors, prefix + name)

    def prepare(self, pack_weights: bool) -> None:
        for part, _ in self._parts():
            part.prepare(pack_weights)

    def forward(self, resid: torch.Tensor, delta: torch.Tensor | None, step: StepContext, cache,
                dtype: torch.dtype) -> torch.Tensor:
        """resid float32 [T, hidden], updated in place; returns the delta still to be added (None if the
        feed-forward added its result itself)."""
        a = self.mixer.forward(NormedInput(self.norm_in, resid, delta, dtype), step, cache, residual=resid)
        return self.ffn.forward(NormedInput(self.norm_post, resid, a, dtype), step, residual=resid)
