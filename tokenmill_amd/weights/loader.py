"""Weights from safetensors files, read by tensor name.

The reference streams every tensor of every ``*.safetensors`` file of the folder by name and then
checks that nothing is missing (reference src/infer/model/loader.py:72-94).  Here the model says
which tensors it expects (name -> shape); the loader checks ALL of them before it moves a byte and
reports everything that is wrong in one error: missing names, unexpected names, wrong shapes.

Storage types: floating tensors are kept in bfloat16, except that a tensor the checkpoint stores
in 32-bit stays 32-bit; integer tables become int32.  With ``dtype="float32"`` (the true 32-bit
path) every floating tensor is widened to 32-bit.
"""
from __future__ import annotations

import fnmatch
import glob
from dataclasses import dataclass
from pathlib import Path

import torch
from safetensors import safe_open


@dataclass(frozen=True)
class TensorSpec:
    """One tensor a model expects in its checkpoint."""
    shape: tuple[int, ...]
    kind: str = "float"          # "float" | "int"
    init: str = "normal"         # random-weights mode: "normal" | "ones" | "zeros" | "index"


class WeightsError(RuntimeError):
    """The checkpoint does not match the model; the message lists every mismatch."""

    def __init__(self, where, missing=(), unexpected=(), wrong_shape=(), other: str | None = None):
        self.missing = sorted(missing)
        self.unexpected = sorted(unexpected)
        self.wrong_shape = sorted(wrong_shape)
        lines = [f"checkpoint {where} does not match the model:"]
        if other:
            lines.append(f"  {other}")
        if self.missing:
            lines.append(f"  missing tensors ({len(self.missing)}): " + ", ".join(self.missing))
        if self.unexpected:
            lines.append(f"  unexpected tensors ({len(self.unexpected)}): " + ", ".join(self.unexpected))
        if self.wrong_shape:
            lines.append(f"  wrong shapes ({len(self.wrong_shape)}): " +
                         ", ".join(f"{n}: file {list(got)} != model {list(want)}"
                                   for n, got, want in self.wrong_shape))
        super().__init__("\n".join(lines))


_FLOAT_TYPES = {torch.float32, torch.bfloat16, torch.float16, torch.float64}


def storage_dtype(stored: torch.dtype, kind: str, dtype: torch.dtype) -> torch.dtype:
    """The type a checkpoint tensor is kept in on the device."""
    if kind == "int":
        return torch.int32
    if dtype == torch.float32:
        return torch.float32
    return torch.float32 if stored in (torch.float32, torch.float64) else torch.bfloat16


def read_checkpoint(model_dir, expected: dict[str, TensorSpec], dtype: torch.dtype, device,
                    ignorable: tuple[str, ...] = ()) -> dict[str, torch.Tensor]:
    """All expected tensors of a model folder, on ``device``.

    ``ignorable``: glob patterns of names a checkpoint may hold without the model using them
    (the reference skips ``rotary_emb`` buffers and, for tied models, ``lm_head.weight``:
    reference src/infer/model/loader.py:80-83,117-118).
    """
    model_dir = Path(model_dir)
    files = sorted(glob.glob(str(model_dir / "*.safetensors")))
    if not files:
        raise WeightsError(model_dir, other=f"no .safetensors files in {model_dir}")
    where: dict[str, str] = {}
    unexpected, wrong = [], []
    for file in files:
        with safe_open(file, framework="pt", device="cpu") as f:
            for name in f.keys():
                if name not in expected:
                    if not any(fnmatch.fnmatch(name, pat) for pat in ignorable):
                        unexpected.append(name)
                    continue
                got = tuple(f.get_slice(name).get_shape())
                if got != tuple(expected[name].shape):
                    wrong.append((name, got, tuple(expected[name].shape)))
                where[name] = file
    missing = [n for n in expected if n not in where]
    if missing or unexpected or wrong:
        raise WeightsError(model_dir, missing, unexpected, wrong)
    out: dict[str, torch.Tensor] = {}
    by_file: dict[str, list[str]] = {}
    for name, file in where.items():
        by_file.setdefault(file, []).append(name)
    for file, names in by_file.items():
        with safe_open(file, framework="pt", device="cpu") as f:
            for name in names:
                t = f.get_tensor(name)
                spec = expected[name]
                if spec.kind == "float" and t.dtype not in _FLOAT_TYPES:
                    raise WeightsError(model_dir, other=f"{name} is stored as {t.dtype}, expected a float type")
                if spec.kind == "int" and t.dtype in _FLOAT_TYPES:
                    raise WeightsError(model_dir, other=f"{name} is stored as {t.dtype}, expected an integer type")
                out[name] = t.to(storage_dtype(t.dtype, spec.kind, dtype)).to(device).contiguous()
    return out
