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


class Drawn:
    """The tokens of one step's rows, on their way to the host: ``device`` holds them (int32 [R]) in stream order,
    ``tokens()`` waits for the copy that was asked for behind them and returns them as a list."""

    def __init__(self, device: torch.Tensor, host: torch.Tensor, copied: torch.cuda.Event):
        self.device, self._host, self._copied = device, host, copied

    def tokens(self) -> list[int]:
        self._copied.synchronize()
        return self._host[:self.device.shape[0]].tolist()


class Sampler:
    HOST_BUFFERS = 4          # pinned buffers for the tokens' way back, used in turn (two steps can be in flight)

    def __init__(self, device):
        self.device = device
        self._host: list[torch.Tensor] = []
        self._turn = 0

    def _host_buffer(self, rows: int) -> torch.Tensor:
        """A pinned buffer for ``rows`` tokens; the one whose last use is the longest ago."""
        i = self._turn % self.HOST_BUFFERS
        self._turn += 1
        if len(self._host) <= i:
            self._host.append(torch.empty(max(rows, 256), dtype=torch.int32, pin_memory=True))
        elif self._host[i].numel() < rows:
            self._host[i] = torch.empty(rows, dtype=torch.int32, pin_memory=True)
        return self._host[i]

    @torch.inference_mode()
    def sample(self, logits: torch.Tensor, params: list[SamplingParams], seeds: list[int],
               counters: list[int]) -> list[int]:
        """logits float32 [R, V] on the GPU; one token per row. ``counters[r]`` is the index of the
        token being generated for row r's request."""
        if logits.shape[0] == 0:
            return []
        return self.start(logits, params, seeds, counters).tokens()

    @torch.inference_mode()
    def start(self, logits: torch.Tensor, params: list[SamplingParams], seeds: list[int],
              counters: list[int]) -> Drawn:
        """As ``sample``, without waiting: the kernels and the copy to the host are queued, and the caller asks
        the returned ``Drawn`` for the tokens when it needs them (its ``device`` tensor can feed the next step
        meanwhile)."""
        with profiling.label("sample", lambda: (logits.numel() * 4, 0)):
            out = self._sample(logits, params, seeds, counters)
        host = self._host_buffer(out.shape[0])
        host[:out.shape[0]].copy_(out, non_blocking=True)
        copied = torch.cuda.Event()
        copied.record()
        return Drawn(out, host, copied)

    def _sample(self, logits, params, seeds, counters) -> torch.Tensor:
        R = logits.shape[0]
        out = torch.empty(R, dtype=torch.int32, device=logits.device)
        if all(p.greedy for p in params):
            ops.argmax_rows(logits, out)
            return out
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
        return out
