"""Greedy, temperature, top-k and top-p sampling over rows of 32-bit logits.

Options and their meanings are the reference's SamplingParams (reference
src/infer/engine/sequence.py:19-31) and sampler (reference src/infer/sampling.py:12-46): argmax for
greedy rows; otherwise logits / temperature, keep the k largest, cut the tail once the mass before a
token exceeds p, softmax, one draw.

The draw itself is this engine's own: the reference gives each request a torch generator so that
its tokens do not depend on its batch-mates (reference src/infer/sampling.py:49-54); here a
request's random number for its n-th generated token is a pure function of (its seed, n), and the
token is the inverse CDF of the filtered softmax in vocabulary order at that number. That is
batch-independent too, and it also survives a preemption that recomputes the request.
"""
from __future__ import annotations

from dataclasses import dataclass, field

import torch

from tokenmill_amd import profiling
from tokenmill_amd.hip import ops

_M64 = (1 << 64) - 1


@dataclass
class SamplingParams:
    max_tokens: int = 256
    temperature: float = 0.0
    top_p: float = 1.0
    top_k: int = -1
    stop: list[str] = field(default_factory=list)      # text-side; kept for interface parity, not used here
    seed: int | None = None
    ignore_eos: bool = False

    @property
    def greedy(self) -> bool:
        return self.temperature <= 1e-5 or self.top_k == 1


def _mix(z: int) -> int:
    z = (z + 0x9E3779B97F4A7C15) & _M64
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & _M64
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & _M64
    return z ^ (z >> 31)


def uniform_from_counter(seed: int, index: int) -> float:
    """u in [0, 1) with 24 random bits for (request seed, index of the generated token)."""
    z = (seed * 0x9E3779B97F4A7C15 + (index + 1) * 0xBF58476D1CE4E5B9) & _M64
    return (_mix(_mix(z)) >> 40) / float(1 << 24)


class Sampler:
    def __init__(self, device):
        self.device = device

    @torch.inference_mode()
    def sample(self, logits: torch.Tensor, params: list[SamplingParams], seeds: list[int],
               counters: list[int]) -> list[int]:
        """logits float32 [R, V] on the GPU; one token per row. ``counters[r]`` is the index of the
        token being generated for row r's request."""
        R = logits.shape[0]
        if R == 0:
            return []
        with profiling.label("sample", lambda: (logits.numel() * 4, 0)):
            return self._sample(logits, params, seeds, counters)

    def _sample(self, logits, params, seeds, counters) -> list[int]:
        R = logits.shape[0]
        out = torch.empty(R, dtype=torch.int32, device=logits.device)
        if all(p.greedy for p in params):
            ops.argmax_rows(logits, out)
            return out.tolist()
        host = torch.empty((4, R), dtype=torch.float32, pin_memory=True)
        host[0] = torch.tensor([p.temperature for p in params])
        host[1] = torch.tensor([p.top_p for p in params])
        host[2] = torch.tensor([0.0 if p.greedy else uniform_from_counter(s, c)
                                for p, s, c in zip(params, seeds, counters)])
        ks = torch.tensor([p.top_k for p in params], dtype=torch.int32).view(torch.float32)
        host[3] = ks                                              # int32 bits travel in the same copy
        dev = host.to(logits.device, non_blocking=True)
        vocab = logits.shape[1]
        ops.sample_rows(logits, dev[0], dev[3].view(torch.int32), dev[1], dev[2], out,
                        uses_top_k=any(not p.greedy and 0 < p.top_k < vocab for p in params),
                        uses_top_p=any(not p.greedy and p.top_p < 1.0 for p in params))
        return out.tolist()
