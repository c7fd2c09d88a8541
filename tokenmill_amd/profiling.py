"""Per-operation GPU time behind a switch, and what a step costs at the least.

Parts mark their device work with ``label(name, bytes, flops)``. Switched off (the default) a label
is a shared no-op. Inside ``collect()`` every label opens a profiler range; the profiler projects a
range onto the GPU's timeline as the span of the kernels launched inside it, so the time of each
operation comes from the device's own clock, not from host timers around launches. With the bytes
an operation has to move and the flops it has to do, the time it could not go below is known, and
the report gives each operation's share of that floor.

The reference's profiler does the same at the level of kernel names: it sorts a profiled decode
step's kernels into buckets and reports the rest of the wall time as "GPU idle"
(reference bench/profile_decode.py:25-41,73-82).
"""
from __future__ import annotations

import contextlib
from dataclasses import dataclass, field

# MI355X data-sheet peaks: HBM3E bytes/s; dense matrix-unit flops/s by compute type
PEAK_HBM_BYTES_S = 8.0e12
PEAK_FLOPS_S = {"bfloat16": 2.5e15, "float32": 157.3e12}

PREFIX = "tm::"


class _Off:
    def __enter__(self):
        return self

    def __exit__(self, *exc):
        return False


_OFF = _Off()
_active: "Collector | None" = None


@dataclass
class OpCost:
    calls: int = 0
    bytes: float = 0.0
    flops: float = 0.0
    device_us: float = 0.0


@dataclass
class Collector:
    ops: dict[str, OpCost] = field(default_factory=dict)
    depth: int = 0
    trace: bool = True


class _Range:
    """An open label: a profiler range (when the GPU is traced), and the mark that labels opened inside
    it belong to it."""

    def __init__(self, collector: Collector, name: str):
        self.collector, self.range = collector, None
        if collector.trace:
            from torch.profiler import record_function
            self.range = record_function(PREFIX + name)

    def __enter__(self):
        self.collector.depth += 1
        if self.range is not None:
            self.range.__enter__()
        return self

    def __exit__(self, *exc):
        if self.range is not None:
            self.range.__exit__(*exc)
        self.collector.depth -= 1
        return False


def label(name: str, cost=None):
    """Marks the device work launched inside as operation ``name``. ``cost``: a function that returns
    (bytes the operation has to move, flops it has to do); it is only called while a ``collect()`` is
    open, and outside one a label costs nothing. A label opened inside another one is part of the outer
    operation (a norm that runs inside the product it feeds), so the operations' times add up."""
    if _active is None or _active.depth > 0:
        return _OFF
    op = _active.ops.setdefault(name, OpCost())
    op.calls += 1
    if cost is not None:
        moved, flops = cost()
        op.bytes += moved
        op.flops += flops
    return _Range(_active, name)


def nbytes(*tensors) -> int:
    """Bytes of the given tensors (None is skipped; a packed matrix counts once)."""
    total = 0
    for t in tensors:
        if t is not None:
            total += t.numel() * t.element_size()
    return total


def on() -> bool:
    return _active is not None


@contextlib.contextmanager
def collect(trace: bool = True):
    """Inside, labels are counted with their costs and, with ``trace``, the GPU is traced. Yields a dict
    that is filled when the block ends: "ops": {name: OpCost}, and with ``trace`` also "kernel_us" (the
    sum over all kernels and copies) and "kernels": {kernel name: us}."""
    global _active
    if _active is not None:
        raise RuntimeError("a profile is already being collected")
    collector = Collector(trace=trace)
    result: dict = {"ops": collector.ops}
    _active = collector
    if not trace:
        try:
            yield result
        finally:
            _active = None
        return
    import torch
    from torch.profiler import ProfilerActivity, profile
    try:
        with profile(activities=[ProfilerActivity.CPU, ProfilerActivity.CUDA]) as prof:
            yield result
            torch.cuda.synchronize()
    finally:
        _active = None
    kernels: dict[str, float] = {}
    total = 0.0
    for evt in prof.events():
        device_us = float(getattr(evt, "device_time_total", 0.0) or 0.0)
        if evt.name.startswith(PREFIX):
            if device_us > 0 and evt.cpu_time_total == 0:          # the range as projected on the GPU's timeline
                collector.ops[evt.name[len(PREFIX):]].device_us += device_us
        elif evt.device_type == torch.autograd.DeviceType.CUDA:
            kernels[evt.name] = kernels.get(evt.name, 0.0) + device_us
            total += device_us
    result.update(kernel_us=total, kernels=kernels)


def floor_us(op: OpCost, dtype_name: str) -> float:
    """The time the operation's calls cannot go below: its bytes at the HBM peak or its flops at the
    matrix-unit peak, whichever is longer."""
    return 1e6 * max(op.bytes / PEAK_HBM_BYTES_S, op.flops / PEAK_FLOPS_S[dtype_name])
