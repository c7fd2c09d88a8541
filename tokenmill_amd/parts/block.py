"""The arrangement of parts in a layer.

PreNormBlock: h = x + mixer(norm_in(x)); y = h + ffn(norm_post(h))
(reference src/infer/model/qwen2.py:13-23). The residual stream is a 32-bit tensor that the
block updates in place; each add is fused into the norm that follows it, so a block takes the
not-yet-added output of the previous block (``delta``) and returns its own.
"""
from __future__ import annotations

import torch

from tokenmill_amd.parts.base import Block, FeedForward, Mixer, Norm, NormedInput, StepContext


class PreNormBlock(Block):
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

    def emit(self, program, cache) -> None:
        """The block as two operations of a step program; a mixer or feed-forward the kernel library has no
        operation for runs through its own ``forward`` between the library's operations."""
        if self.mixer.emit(program, self.norm_in, cache) is None:
            def mix(flow, step):
                x = NormedInput(self.norm_in, flow.resid, flow.delta, program.dtype)
                flow.delta = self.mixer.forward(x, step, cache, residual=flow.resid)
                assert x.delta is None, f"{type(self.mixer).__name__}.forward did not take its input"
            program.foreign(self.mixer, mix)
        if self.ffn.emit(program, self.norm_post) is None:
            def feed(flow, step):
                x = NormedInput(self.norm_post, flow.resid, flow.delta, program.dtype)
                flow.delta = self.ffn.forward(x, step, residual=flow.resid)
                assert x.delta is None, f"{type(self.ffn).__name__}.forward did not take its input"
            program.foreign(self.ffn, feed)

    def forward(self, resid: torch.Tensor, delta: torch.Tensor | None, step: StepContext, cache,
                dtype: torch.dtype) -> torch.Tensor:
        """resid float32 [T, hidden], updated in place; returns the delta still to be added (None if the
        feed-forward added its result itself)."""
        a = self.mixer.forward(NormedInput(self.norm_in, resid, delta, dtype), step, cache, residual=resid)
        return self.ffn.forward(NormedInput(self.norm_post, resid, a, dtype), step, residual=resid)
