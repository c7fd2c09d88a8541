"""Random-weights mode: write a model folder (config.json, model.safetensors) from a
configuration and a seed.

The reference has no such mode (its tests build a tiny model through another library and its
benchmarks load a real checkpoint: reference tests/conftest.py:52-64).  Which tensors exist, and
their shapes, come from the architecture's own model through the registry, so this file knows no
architecture.  Each tensor is drawn from a generator keyed by (seed, tensor name): any one tensor
can be reproduced without drawing the others.

    python -m tokenmill_amd.weights.random_init --config config.json --seed 0 --out DIR
"""
from __future__ import annotations

import argparse
import hashlib
import json
from pathlib import Path
from typing import Iterator

import torch

from tokenmill_amd.weights.loader import TensorSpec


def _generator(seed: int, name: str) -> torch.Generator:
    digest = hashlib.sha256(f"{seed}:{name}".encode()).digest()
    return torch.Generator().manual_seed(int.from_bytes(digest[:8], "little") >> 1)


def random_tensors(specs: dict[str, TensorSpec], seed: int, std: float = 0.02, norm_std: float = 0.0,
                   storage: torch.dtype = torch.bfloat16) -> Iterator[tuple[str, torch.Tensor]]:
    """(name, tensor) for every spec: "normal" ~ N(0, std); "ones" = 1 + N(0, norm_std)."""
    for name in sorted(specs):
        spec = specs[name]
        g = _generator(seed, name)
        if spec.kind == "int":
            t = torch.arange(int(torch.tensor(spec.shape).prod()), dtype=torch.int32).reshape(spec.shape)
        elif spec.init == "ones":
            t = torch.ones(spec.shape, dtype=torch.float32)
            if norm_std:
                t += torch.randn(spec.shape, generator=g, dtype=torch.float32) * norm_std
            t = t.to(storage)
        elif spec.init == "zeros":
            t = torch.zeros(spec.shape, dtype=storage)
        else:
            t = (torch.randn(spec.shape, generator=g, dtype=torch.float32) * std).to(storage)
        yield name, t


def write_random_model(config: dict, out_dir, seed: int, std: float = 0.02, norm_std: float = 0.0,
                       storage: str = "bfloat16") -> Path:
    """Write ``config.json`` and ``model.safetensors`` for the architecture that ``config`` names."""
    from safetensors.torch import save_file

    from tokenmill_amd.config.registry import architecture_name, get_architecture

    arch = get_architecture(architecture_name(config))
    cfg = arch.config_from_dict(config, None)
    model = arch.build_model(cfg)
    dt = {"bfloat16": torch.bfloat16, "float32": torch.float32}[storage]
    tensors = dict(random_tensors(model.tensor_specs(), seed, std, norm_std, dt))
    out_dir = Path(out_dir)
    out_dir.mkdir(parents=True, exist_ok=True)
    (out_dir / "config.json").write_text(json.dumps(config, indent=1))
    save_file(tensors, str(out_dir / "model.safetensors"))
    return out_dir


def main(argv=None) -> None:
    p = argparse.ArgumentParser(description="write a model folder with random weights")
    p.add_argument("--config", required=True,
                   help="a config.json of a registered architecture, or a shipped shape's name (tiny-a, 0.5b, 7b, ...)")
    p.add_argument("--out", required=True)
    p.add_argument("--seed", type=int, default=0)
    p.add_argument("--std", type=float, default=0.02)
    p.add_argument("--norm-std", type=float, default=0.0, help="norm weights are 1 + N(0, this)")
    p.add_argument("--storage", default="bfloat16", choices=["bfloat16", "float32"])
    a = p.parse_args(argv)
    from tokenmill_amd.config.shapes import read_shape

    write_random_model(read_shape(a.config), a.out, a.seed, a.std, a.norm_std, a.storage)
    print(f"wrote {a.out}")


if __name__ == "__main__":
    main()
