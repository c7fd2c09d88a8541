"""A model's step as a few calls into the kernel library.

Every part describes its operation to a ``StepProgram`` once, at engine start (``Part.emit``): the
embedding, for every run call a pre-norm attention operation and a pre-norm feed-forward operation with
their matrices, norms, rotary tables and cache pools, the final norm with the output head. Operations the
library has (``csrc/step_program.hip``) are appended to the program there; a part the library has no
operation for (a mixer with state, a routed feed-forward, another position encoding or norm) is kept as a
call of its own ``forward``. ``run(step)`` then walks the list: consecutive library operations are ONE call
(which chooses and launches their kernels), a foreign part is a hop back to its own code, and the
residual stream with the not-yet-added result of the last product crosses from one to the next. So there
is one forward pass, whichever parts a model has, and one foreign part costs one hop, not the model.

A part that is called by itself (by a foreign block's code, or a test) runs a one-operation program of its
own through the same entry, so the rules that choose kernels exist once, inside the library.
"""
from __future__ import annotations

import ctypes
import weakref
from dataclasses import dataclass
from typing import TYPE_CHECKING, Callable

import torch

from tokenmill_amd import profiling
from tokenmill_amd.hip import abi, ops
from tokenmill_amd.hip.abi import TmAttentionOp, TmEmbedOp, TmFfnOp, TmFinalOp, TmLinear, TmNorm, TmStep, TmStream

if TYPE_CHECKING:
    from tokenmill_amd.parts.base import StepContext


@dataclass
class Flow:
    """What crosses from one operation of a step to the next."""
    resid: torch.Tensor | None = None        # float32 [T, hidden], the residual stream
    delta: torch.Tensor | None = None        # a result [T, hidden] still to be added to it
    logits: torch.Tensor | None = None       # float32 [R, vocab], set by the head
    x: torch.Tensor | None = None            # into a single operation: its input, already normed
    qkv: torch.Tensor | None = None          # into a single attention: q|k|v already projected, encoded and stored
    accumulate: bool = True                  # may an operation add its result into resid itself?


@dataclass
class _Native:
    first: int
    count: int


@dataclass
class _Foreign:
    part: object
    fn: Callable[[Flow, "StepContext"], None]


_live: "weakref.WeakValueDictionary[int, StepProgram]" = weakref.WeakValueDictionary()     # by the number their hook is called with


def _on_label(user, op, label, begin):
    program = _live.get(user)
    if program is not None:
        program._label(op, abi.LABELS[label], bool(begin))


_HOOK = abi.TmHook(_on_label)
_numbers = iter(range(1, 1 << 62))


class StepProgram:
    def __init__(self, dtype: torch.dtype, hidden: int, device, tune: tuple[int, bool] | None = None):
        self._lib = abi.bound()
        self.dtype, self.hidden, self.device = dtype, hidden, torch.device(device)
        self._handle = self._lib.tm_program_create(ops.code(dtype), hidden)
        if not self._handle:
            raise ops.KernelArgumentError(f"the kernel library runs no program of {dtype} and width {hidden}")
        self.tune = tune if tune and tune[0] >= 2 else None       # (candidates, every): this program's products are timed
        if self.tune and self._lib.tm_program_set_tune(self._handle, int(self.tune[0]), 1 if self.tune[1] else 0):
            raise ops.KernelArgumentError(f"tune: {self.tune}")
        self._number = next(_numbers)
        self._lib.tm_program_set_hook(self._handle, _HOOK, self._number)
        _live[self._number] = self
        self.steps: list[_Native | _Foreign] = []
        self.parts: list[object] = []            # by operation index: the part that described it
        self._keep: list[object] = []            # every tensor the library's operations point at
        self.vocab: int | None = None
        self.runs = 0
        self._now: tuple | None = None           # (step, rows) of the run in flight, for the labels' costs
        self._open: list = []

    def __del__(self):
        if getattr(self, "_handle", None):
            self._lib.tm_program_destroy(self._handle)
            self._handle = None

    # --- described by the parts ---------------------------------------------------------------------------

    def _norm(self, norm) -> TmNorm | None:
        """``norm`` as the library takes it; a null norm for None (the operation is always handed its input normed);
        None for a norm the library does not compute."""
        if norm is None:
            return TmNorm(None, -1, 0.0)
        params = norm.rms_params()
        if params is None or params[0] is None:
            return None
        self._keep.append(params[0])
        return TmNorm(params[0].data_ptr(), ops.code(params[0].dtype), float(params[1]))

    def _linear(self, lin) -> TmLinear | None:
        desc = lin.describe()
        if desc is None:
            return None
        self._keep.append((lin.weight, lin.bias, lin.packed))
        return desc

    def _added(self, index: int, part) -> int | None:
        if index < 0:
            return None
        assert index == len(self.parts)
        self.parts.append(part)
        if self.steps and isinstance(self.steps[-1], _Native) and self.steps[-1].first + self.steps[-1].count == index:
            self.steps[-1].count += 1
        else:
            self.steps.append(_Native(index, 1))
        return index

    def embedding(self, part, table: torch.Tensor) -> int | None:
        """resid = table[token_ids]. Returns the operation's index, or None if the library does not run it."""
        if table is None or not table.is_cuda or table.dim() != 2 or table.shape[1] != self.hidden or not table.is_contiguous() \
                or table.dtype not in (torch.float32, torch.bfloat16):
            return None
        self._keep.append(table)
        op = TmEmbedOp(table.data_ptr(), ops.code(table.dtype), table.shape[0], self.hidden)
        return self._added(self._lib.tm_program_add_embedding(self._handle, ctypes.byref(op)), part)

    def attention(self, part, norm, qkv, o, rotation, cache, num_heads: int, num_kv_heads: int, head_dim: int,
                  scale: float, window: int | None) -> int | None:
        """resid += o(attention(rotate(qkv(norm(resid))))) over the paged cache ``cache`` (a ``KVCacheView``).
        ``rotation``: (cos, sin, rotary width, positions) of a rotary encoding, or () for none."""
        n, q, out = self._norm(norm), self._linear(qkv), self._linear(o)
        if n is None or q is None or out is None or getattr(cache, "k", None) is None:
            return None
        if rotation:
            cos, sin, rot, n_pos = rotation
            self._keep.append((cos, sin))
            cos, sin = cos.data_ptr(), sin.data_ptr()
        else:
            cos = sin = None
            rot = n_pos = 0
        self._keep.append((cache.k, cache.v))
        op = TmAttentionOp(n, q, out, cos, sin, cache.k.data_ptr(), cache.v.data_ptr(), num_heads, num_kv_heads, head_dim,
                           float(scale), window or 0, rot, n_pos, cache.k.shape[1], cache.group, 1 if cache.write else 0)
        return self._added(self._lib.tm_program_add_attention(self._handle, ctypes.byref(op)), part)

    def feed_forward(self, part, norm, gate_up, down, intermediate: int) -> int | None:
        """resid += down(silu(gate(n)) * up(n)), n = norm(resid); gate and up stacked in one matrix."""
        n, gu, dn = self._norm(norm), self._linear(gate_up), self._linear(down)
        if n is None or gu is None or dn is None:
            return None
        op = TmFfnOp(n, gu, dn, intermediate)
        return self._added(self._lib.tm_program_add_feed_forward(self._handle, ctypes.byref(op)), part)

    def head(self, part, norm, proj, vocab: int) -> int | None:
        """logits = proj(norm(resid[logit rows])) in float32."""
        n, h = self._norm(norm), self._linear(proj)
        if n is None or h is None:
            return None
        index = self._added(self._lib.tm_program_add_head(self._handle, ctypes.byref(TmFinalOp(n, h))), part)
        if index is not None:
            self.vocab = vocab
        return index

    def foreign(self, part, fn: Callable[[Flow, "StepContext"], None]) -> None:
        """A part the library has no operation for: ``fn(flow, step)`` runs it through its own code."""
        self.steps.append(_Foreign(part, fn))

    @property
    def foreign_parts(self) -> list[object]:
        return [s.part for s in self.steps if isinstance(s, _Foreign)]

    # --- run -------------------------------------------------------------------------------------------------

    def counters(self) -> dict[str, int]:
        """How often each way of computing q|k|v and the feed-forward's activation has been taken."""
        out = (ctypes.c_longlong * len(abi.COUNTERS))()
        self._lib.tm_program_counters(self._handle, out)
        return dict(zip(abi.COUNTERS, out))

    def _label(self, op: int, name: str, begin: bool) -> None:
        """Called by the library around a span's launches while a profile is collected."""
        if begin:
            step, rows = self._now
            part = self.parts[op]
            ctx = profiling.label(name, lambda: part.cost(name, step, rows))
            ctx.__enter__()
            self._open.append(ctx)
        elif self._open:
            self._open.pop().__exit__(None, None, None)

    @staticmethod
    def _step_struct(step: "StepContext | None", rows: int) -> TmStep:
        s = TmStep()
        if step is None:                          # an operation that looks at no token's position or request
            s.T = rows
            return s
        s.T, s.S, s.R, s.num_decode = step.num_tokens, step.num_seqs, step.num_logit_rows, step.num_decode
        s.max_context_len, s.max_decode_context = step.max_context_len, step.max_decode_context
        tiles = step.prefill_tiles
        s.n_tiles = tiles.shape[0] if tiles is not None else 0
        s.prefill_tiles = tiles.data_ptr() if s.n_tiles else None
        if len(step.groups) > abi.MAX_GROUPS:
            raise ops.KernelArgumentError(f"a step of {len(step.groups)} cache groups; the library takes {abi.MAX_GROUPS}")
        s.num_groups = len(step.groups)
        s.token_ids, s.positions = step.token_ids.data_ptr(), step.positions.data_ptr()
        s.seq_of_token, s.context_lens = step.seq_of_token.data_ptr(), step.context_lens.data_ptr()
        s.logit_rows = step.logit_rows.data_ptr() if s.R else None
        for g, group in enumerate(step.groups):
            s.block_tables[g] = group.block_tables.data_ptr()
            s.slot_mapping[g] = group.slot_mapping.data_ptr()
            s.table_width[g] = group.block_tables.shape[1]
        return s

    def run_ops(self, first: int, count: int, step: "StepContext | None", flow: Flow, rows: int | None = None,
                at_once: bool = False, _shared: dict | None = None) -> None:
        """Operations [first, first + count) as one call into the library. ``flow`` is updated in place: its delta
        becomes what the last operation left to be added (a view of this call's workspace) or None."""
        T = step.num_tokens if step is not None else rows
        R = step.num_logit_rows if step is not None else 0
        nd = step.num_decode if step is not None else 0
        shared = _shared if _shared is not None else {}
        if "struct" not in shared:
            shared["struct"] = self._step_struct(step, T)
            need = self._lib.tm_program_workspace_bytes(self._handle, T, R, nd, step.max_decode_context if step is not None else 0)
            shared["workspace"] = torch.empty(need, dtype=torch.uint8, device=self.device)
        workspace = shared["workspace"]
        io = TmStream()
        for name in ("resid", "delta", "x", "qkv"):
            t = getattr(flow, name)
            if t is not None:
                if not t.is_cuda or not t.is_contiguous():
                    raise ops.KernelArgumentError(f"the step program takes contiguous tensors on the GPU ({name})")
                setattr(io, name, t.data_ptr())
        if flow.resid is not None and (flow.resid.dtype != torch.float32 or tuple(flow.resid.shape) != (T, self.hidden)):
            raise ops.KernelArgumentError(f"the residual stream must be float32 [{T}, {self.hidden}]")
        for name in ("delta", "x"):
            t = getattr(flow, name)
            if t is not None and (t.dtype != self.dtype or tuple(t.shape) != (T, self.hidden)):
                raise ops.KernelArgumentError(f"{name} must be {self.dtype} [{T}, {self.hidden}]")
        io.accumulate = 1 if flow.accumulate and flow.resid is not None else 0
        flags = (abi.RUN_LABELS if profiling.on() else 0) | (abi.RUN_TUNE_AT_ONCE if at_once else 0)
        lib_ws = ops.library_workspace(self.device)
        self._now = (step, T)
        try:
            rc = self._lib.tm_program_run(self._handle, first, count, ctypes.byref(shared["struct"]), ctypes.byref(io),
                                          workspace.data_ptr(), workspace.numel(), lib_ws.data_ptr(),
                                          ops.LIBRARY_WORKSPACE_BYTES, flow.logits.data_ptr() if flow.logits is not None else None,
                                          flags, ops._stream())
        finally:
            self._now = None
            while self._open:                                   # a run that failed inside a span
                self._open.pop().__exit__(None, None, None)
        if rc == 1:
            raise ops.KernelArgumentError("the step program refused the step (a size or position a kernel does not run)")
        if rc != 0:
            raise RuntimeError(f"the step program failed (code {rc})")
        flow.x = flow.qkv = None
        if io.delta:
            off = io.delta - workspace.data_ptr()
            n = T * self.hidden * torch.empty((), dtype=self.dtype).element_size()
            flow.delta = workspace[off:off + n].view(self.dtype).view(T, self.hidden)
        else:
            flow.delta = None

    def run(self, step: "StepContext", at_once: bool = False) -> torch.Tensor:
        """The step's float32 logits [R, vocab] at ``step.logit_rows``. ``at_once``: library products time their
        algorithms at this call, if this program times at all (the step is about to be captured into a graph)."""
        T, R = step.num_tokens, step.num_logit_rows
        flow = Flow(resid=torch.empty((T, self.hidden), dtype=torch.float32, device=self.device))
        if self.vocab is not None:
            flow.logits = torch.empty((R, self.vocab), dtype=torch.float32, device=self.device)
        shared: dict = {}
        for st in self.steps:
            if isinstance(st, _Native):
                self.run_ops(st.first, st.count, step, flow, at_once=at_once, _shared=shared)
            elif self.tune:
                with ops.tuning(self.tune[0], 1 if at_once else ops.TUNE_AFTER_CALLS, self.tune[1]):
                    st.fn(flow, step)
            else:
                st.fn(flow, step)
        self.runs += 1
        if flow.logits is None:
            raise RuntimeError("the model's last part set no logits")
        return flow.logits

    def run_one(self, op: int, step: "StepContext | None", *, resid=None, delta=None, x=None, qkv=None,
                accumulate: bool = False, rows: int | None = None) -> torch.Tensor | None:
        """One operation by itself (a part called from outside a program). Returns what it left to be added to the
        residual stream, or None if it added that itself (``accumulate``)."""
        flow = Flow(resid=resid, delta=delta, x=x, qkv=qkv, accumulate=accumulate)
        self.run_ops(op, 1, step, flow, rows=rows)
        return flow.delta
