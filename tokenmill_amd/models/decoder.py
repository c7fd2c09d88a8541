"""A decoder made of parts: embedding, a list of layers, the order in which they run, a final
norm and an output head. It knows no architecture; an architecture is a function that fills it.

The order in which layers run is data: ``run`` is a list of ``LayerCall``. A layer may be named
more than once (it then runs again with the same weights), and a call may read the cache that an
earlier call writes instead of having one of its own.
"""
from __future__ import annotations

from dataclasses import dataclass

import torch

from tokenmill_amd.parts.base import KVCacheSpec, Norm, Part, StateSpec
from tokenmill_amd.weights.loader import TensorSpec


@dataclass(frozen=True)
class LayerCall:
    layer: int                       # index into DecoderModel.layers
    cache_of: int | None = None      # None: this call has a cache of its own; j: it reads the cache of run[j]


class DecoderModel:
    def __init__(self, config, embedding: Part, layers: list, final_norm: Norm, head: Part,
                 run: list[LayerCall] | None = None,
                 names: tuple[str, str, str, str] = ("model.embed_tokens.", "model.layers.{i}.", "model.norm.", ""),
                 ignorable: tuple[str, ...] = ()):
        self.config = config
        self.embedding, self.layers, self.final_norm, self.head = embedding, layers, final_norm, head
        self.run = run if run is not None else [LayerCall(i) for i in range(len(layers))]
        self.names = names
        self.ignorable = ignorable
        self.dtype: torch.dtype | None = None
        self.device = None
        for j, call in enumerate(self.run):
            if not 0 <= call.layer < len(layers):
                raise ValueError(f"run[{j}] names layer {call.layer}; the model has {len(layers)}")
            if call.cache_of is not None:
                if not 0 <= call.cache_of < j or self.run[call.cache_of].cache_of is not None:
                    raise ValueError(f"run[{j}] must read the cache of an earlier call that owns one")
                if layers[call.layer].mixer.cache_spec() != layers[self.run[call.cache_of].layer].mixer.cache_spec():
                    raise ValueError(f"run[{j}] reads a cache of another geometry than its own mixer's")

    # --- tensors ---------------------------------------------------------------------------------

    def _prefixed(self):
        emb, layer, norm, head = self.names
        yield self.embedding, emb
        for i, block in enumerate(self.layers):
            yield block, layer.format(i=i)
        yield self.final_norm, norm
        yield self.head, head

    def tensor_specs(self) -> dict[str, TensorSpec]:
        specs: dict[str, TensorSpec] = {}
        for part, prefix in self._prefixed():
            specs.update(part.tensor_specs(prefix))
        return specs

    def load(self, tensors: dict[str, torch.Tensor], dtype: torch.dtype, device, pack_weights: bool = True) -> None:
        """Every part takes its tensors, then prepares what its kernels want beside them."""
        self.dtype, self.device = dtype, device
        for part, prefix in self._prefixed():
            part.load(tensors, prefix)
        for part, _ in self._prefixed():
            part.prepare(pack_weights)

    # --- what the cache manager must provide -------------------------------------------------------

    def cache_specs(self) -> list[KVCacheSpec | StateSpec | None]:
        """One entry per run call: the cache its mixer needs, or None for a call that reads another's."""
        return [None if c.cache_of is not None else self.layers[c.layer].mixer.cache_spec() for c in self.run]

    # --- one step -----------------------------------------------------------------------------------

    def program(self, caches: list, tune: tuple[int, bool] | None = None):
        """The model's step as a ``StepProgram``: every part describes its operation to it, in the order of the
        run list; ``caches[j]`` is the cache view of run call j (shared ones resolved). Running the program on
        a step gives the float32 logits [R, vocab] at ``step.logit_rows``. A part the kernel library has no
        operation for is called through its own ``forward`` at its place. ``tune``: (candidates, every) if the
        library's matrix products are to be timed for this model's steps."""
        from tokenmill_amd.hip.program import StepProgram
        program = StepProgram(self.dtype, self.embedding.hidden, self.device, tune)
        emb, head, norm = self.embedding, self.head, self.final_norm
        if getattr(emb, "emit", lambda p: None)(program) is None:
            def embed(flow, step):
                flow.resid, flow.delta = emb.forward(step.token_ids), None
            program.foreign(emb, embed)
        for j, call in enumerate(self.run):
            self.layers[call.layer].emit(program, caches[j])
        if getattr(head, "emit", lambda p, n: None)(program, norm) is None:
            def logits(flow, step):
                if step.num_logit_rows == 0:
                    flow.logits = torch.empty((0, head.vocab), dtype=torch.float32, device=flow.resid.device)
                else:
                    flow.logits = head.forward(norm.add_norm(flow.resid, flow.delta, self.dtype, rows=step.logit_rows))
                flow.delta = None
            program.foreign(head, logits)
        return program
