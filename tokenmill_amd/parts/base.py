"""What every part of a layer looks like to the model that holds it.

A part (mixer, feed-forward, norm, position encoding, embedding, output head) gets its sizes and
constants as constructor parameters, declares the checkpoint tensors it wants under a prefix,
takes them in ``load`` and computes in ``forward``. No part knows which model it is in.

Per step, every part sees the same ``StepContext``: the flat batch of tokens with each token's
absolute position and request, and per cache group the block tables and slot mapping.
"""
from __future__ import annotations

from dataclasses import dataclass, field

import torch

from tokenmill_amd.weights.loader import TensorSpec


# ------------------------------------------------------------------------------------------------
# what a mixer asks of the cache manager
# ------------------------------------------------------------------------------------------------

@dataclass(frozen=True)
class KVCacheSpec:
    """Keys and values in pages. ``window``: None keeps every token; W keeps the last W."""
    kv_heads: int
    head_dim: int
    window: int | None = None


@dataclass(frozen=True)
class StateSpec:
    """State of fixed size per request (zeroed when a request is admitted)."""
    shape: tuple[int, ...]
    dtype: torch.dtype = torch.float32


@dataclass
class KVCacheView:
    """One cache layer as a mixer sees it."""
    k: torch.Tensor              # [pages, page_size, kv_heads, head_dim]
    v: torch.Tensor              # [pages, kv_heads, head_dim, page_size]
    group: int                   # index into StepContext.groups
    write: bool = True           # False: this layer reads a cache that another layer writes


@dataclass
class StateView:
    state: torch.Tensor          # [slots, *shape]; row StepContext.state_slots[s] belongs to request s


# ------------------------------------------------------------------------------------------------
# the step as parts see it
# ------------------------------------------------------------------------------------------------

@dataclass
class GroupStep:
    block_tables: torch.Tensor   # int32 [S, W]: page ids of each request of the step, in this group
    slot_mapping: torch.Tensor   # int32 [T]: flat cache slot of each token of the step, in this group


@dataclass
class StepContext:
    num_tokens: int
    num_seqs: int
    token_ids: torch.Tensor      # int32 [T]
    positions: torch.Tensor      # int32 [T]  absolute position of each token in its own request
    seq_of_token: torch.Tensor   # int32 [T]  index of the token's request in this step
    cu_q_lens: torch.Tensor      # int32 [S+1] first row of each request's tokens
    context_lens: torch.Tensor   # int32 [S]  tokens of the request once this step is done
    state_slots: torch.Tensor    # int32 [S]
    logit_rows: torch.Tensor     # int32 [R]  rows whose logits are wanted
    groups: list[GroupStep] = field(default_factory=list)
    # host-side copies for choosing kernels and grids
    q_lens: list[int] = field(default_factory=list)
    start_positions: list[int] = field(default_factory=list)
    max_q_len: int = 0
    max_context_len: int = 0
    num_logit_rows: int = 0
    # S entries are ordered with the q_len == 1 entries last; this many of them:
    num_decode: int = 0
    max_decode_context: int = 0      # longest context among them (new token counted)
    # the q_len > 1 entries cut into tiles of at most 16 tokens: int32 [n, 4] =
    # (request index, first row, tokens, position of the first token)
    prefill_tiles: torch.Tensor | None = None


# ------------------------------------------------------------------------------------------------
# the part interfaces
# ------------------------------------------------------------------------------------------------

class Part:
    """Base of all parts: declares tensors, takes them, computes."""

    def tensor_specs(self, prefix: str) -> dict[str, TensorSpec]:
        """Checkpoint tensors this part expects, by full name."""
        return {}

    def load(self, tensors: dict[str, torch.Tensor], prefix: str) -> None:
        """Take this part's tensors (already on the device, in their storage type)."""

    def prepare(self, pack_weights: bool) -> None:
        """Called once after ``load``: make what the kernels want beside the checkpoint's tensors.
        ``pack_weights``: whether second copies of matrices in a kernel's own order may be kept."""

    def cost(self, label: str, step: "StepContext | None", rows: int) -> tuple[int, int]:
        """(bytes, flops) that the span ``label`` of this part's operation has to move and do for a step of
        ``rows`` tokens: what a profile prices the span's measured time against. Only parts that describe an
        operation to the step program are asked."""
        return 0, 0


class Norm(Part):
    def add_norm(self, resid: torch.Tensor, delta: torch.Tensor | None, out_dtype: torch.dtype,
                 rows: torch.Tensor | None = None) -> torch.Tensor:
        """resid (float32 [T, hidden]) += delta, in place; returns norm(resid) in ``out_dtype``.
        With ``rows``: only those rows, and resid is left as it is."""
        raise NotImplementedError

    def rms_params(self) -> tuple[torch.Tensor, float] | None:
        """(weight, eps) if this norm is weight * round(x * rsqrt(mean(x^2) + eps)), which kernels that
        follow it can compute themselves; None for any other norm."""
        return None


class NormedInput:
    """The input of a mixer or feed-forward that is still to be computed: norm(resid + delta).

    A part either calls ``tensor()`` (the add and the norm run as one kernel; resid is updated in
    place) or, if it has a kernel that starts with the norm, takes ``fusable_rms()`` and reads
    ``resid`` itself. One of the two must happen, or a pending delta would be lost."""

    def __init__(self, norm: Norm, resid: torch.Tensor, delta: torch.Tensor | None, dtype: torch.dtype):
        self.norm, self.resid, self.delta, self.dtype = norm, resid, delta, dtype
        self._tensor: torch.Tensor | None = None
        self.taken = False                   # a kernel that starts at the norm has taken resid and delta as they are

    @property
    def num_tokens(self) -> int:
        return self.resid.shape[0]

    def tensor(self) -> torch.Tensor:
        if self._tensor is None:
            self._tensor = self.norm.add_norm(self.resid, self.delta, self.dtype)
            self.delta = None
        return self._tensor

    def fusable_rms(self) -> tuple[torch.Tensor, float] | None:
        """(weight, eps) when nothing is pending on the residual and the norm is an RMS norm."""
        if self._tensor is not None or self.delta is not None:
            return None
        return self.norm.rms_params()

    @property
    def lazy(self) -> bool:
        """Still to be computed, by a norm the kernel library computes itself?"""
        return self._tensor is None and not self.taken and self.norm.rms_params() is not None

    def take(self) -> tuple[torch.Tensor, torch.Tensor | None]:
        """(resid, delta) for an operation that adds and norms by itself; after this the input counts as computed."""
        self.taken = True
        delta, self.delta = self.delta, None
        return self.resid, delta


def as_tensor(x) -> torch.Tensor:
    """The input of a part as a tensor, whether it came lazily or not."""
    return x.tensor() if isinstance(x, NormedInput) else x


class PositionEncoding(Part):
    def rotation(self):
        """What the kernel library's attention operation needs to apply this encoding itself: (cos, sin, rotary
        width, positions) for a rotation of pairs, () for no encoding at all, None (the default) for an encoding
        the library does not know: the mixer then projects q|k|v, calls ``encode_and_store`` and goes on from there."""
        return None

    def encode_and_store(self, qkv: torch.Tensor, num_heads: int, num_kv_heads: int, head_dim: int,
                         step: StepContext, cache: KVCacheView) -> None:
        """Encode positions into q and k of ``qkv`` in place and store k, v into the cache."""
        raise NotImplementedError


class Mixer(Part):
    def emit(self, program, norm: Norm, cache) -> int | None:
        """Describes ``resid += self(norm(resid))`` over ``cache`` to the step program (``hip/program.py``) and
        returns the operation's index; None (the default) if the kernel library has no operation for this
        mixer: the program then calls ``forward``."""
        return None

    # Can a step of single tokens through this mixer be recorded into a HIP graph? Yes if ``forward`` works on
    # the step's device tensors alone for such a step (index operations with ``state_slots``, kernels);
    # no if it needs their values on the host (``.tolist()``, ``.item()``) or allocates by them. Only asked
    # of mixers with per-request state: their decode steps are then replayed like any other model's.
    capturable = True

    def cache_spec(self) -> KVCacheSpec | StateSpec | None:
        return None

    def forward(self, x, step: StepContext, cache, residual: torch.Tensor | None = None) -> torch.Tensor | None:
        """x: the normed input [T, hidden], as a tensor or a ``NormedInput`` (``as_tensor(x)`` gives the
        tensor). Returns [T, hidden] to be added to the residual stream; or, if ``residual`` (float32
        [T, hidden]) is given, it may add its result there itself and return None."""
        raise NotImplementedError


class FeedForward(Part):
    def emit(self, program, norm: Norm) -> int | None:
        """As ``Mixer.emit``, for ``resid += self(norm(resid))``."""
        return None

    def forward(self, x, step: StepContext, residual: torch.Tensor | None = None) -> torch.Tensor | None:
        """Same contract as ``Mixer.forward``, without a cache."""
        raise NotImplementedError


class Block(Part):
    """An arrangement of parts in a layer. ``forward(resid, delta, step, cache, dtype)`` updates the 32-bit
    residual stream ``resid`` in place, given the not-yet-added result ``delta`` of the block before, and
    returns its own not-yet-added result (or None). ``emit`` describes the block to a step program; by
    default as one call of ``forward``, so a block written elsewhere needs nothing more."""

    mixer: Mixer

    def forward(self, resid: torch.Tensor, delta: torch.Tensor | None, step: StepContext, cache,
                dtype: torch.dtype) -> torch.Tensor | None:
        raise NotImplementedError

    def emit(self, program, cache) -> None:
        def run(flow, step):
            flow.delta = self.forward(flow.resid, flow.delta, step, cache, program.dtype)
        program.foreign(self, run)
