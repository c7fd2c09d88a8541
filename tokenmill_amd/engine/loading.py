"""From a model folder to a model on the GPU (reference src/infer/model/loader.py:32-41,49-95)."""
from __future__ import annotations

from pathlib import Path

import torch

from tokenmill_amd.config.registry import load_config
from tokenmill_amd.weights.loader import read_checkpoint


def resolve_dtype(name: str) -> torch.dtype:
    """auto = bfloat16, the type serving uses (reference src/infer/model/loader.py:32-35 picks the
    16-bit type on a GPU); float32 = the true 32-bit path."""
    try:
        return {"auto": torch.bfloat16, "bfloat16": torch.bfloat16, "float32": torch.float32}[name]
    except KeyError:
        raise ValueError(f"dtype '{name}' is not one of auto, bfloat16, float32") from None


def resolve_device(name: str) -> torch.device:
    """There is no CPU path: the device is a GPU or the call fails."""
    if not torch.cuda.is_available():
        raise RuntimeError("tokenmill_amd needs a GPU (gfx950); none is visible")
    return torch.device("cuda:0" if name == "auto" else name)


def check_positions(model_config, max_positions: int | None) -> None:
    """Refuses, before anything is loaded, a context the model's position tables do not reach: the reference
    sizes its rotary table ``min(max_model_len, max_position_embeddings)`` (reference
    src/infer/model/qwen2.py:34, src/infer/engine/engine.py:94), so a longer context would index beyond it."""
    from tokenmill_amd.config.model_config import ConfigError
    most = getattr(model_config, "max_position_embeddings", None)
    if max_positions is not None and max_positions < 1:
        raise ConfigError(f"max_model_len must be at least 1, got {max_positions}")
    if max_positions is not None and most is not None and max_positions > most:
        raise ConfigError(f"max_model_len {max_positions} exceeds the model's max_position_embeddings {most}")


def load_model(model_dir: str | Path, dtype: torch.dtype, device: torch.device, max_positions: int | None = None,
               pack_weights: bool = True):
    """The model that config.json names, with its weights on ``device``. ``pack_weights``: keep a second
    copy of each layer matrix in the order the decode-step kernels read it."""
    arch, cfg = load_config(model_dir)
    check_positions(cfg, max_positions)
    model = arch.build_model(cfg, max_positions)
    tensors = read_checkpoint(model_dir, model.tensor_specs(), dtype, device, model.ignorable)
    model.load(tensors, dtype, device, pack_weights=pack_weights)
    return model


def load_random_model(config: dict, seed: int, dtype: torch.dtype, device: torch.device,
                      max_positions: int | None = None, std: float = 0.02, norm_std: float = 0.0,
                      pack_weights: bool = True):
    """The model that ``config`` (config.json contents) names, with random weights drawn on the
    device: the random-weights mode without the trip through a file, for large shapes."""
    from tokenmill_amd.config.registry import architecture_name, get_architecture
    from tokenmill_amd.weights.loader import storage_dtype

    arch = get_architecture(architecture_name(config))
    cfg = arch.config_from_dict(config, None)
    check_positions(cfg, max_positions)
    model = arch.build_model(cfg, max_positions)
    g = torch.Generator(device=device).manual_seed(seed)
    tensors = {}
    for name, spec in sorted(model.tensor_specs().items()):
        if spec.kind == "int":
            t = torch.arange(int(torch.tensor(spec.shape).prod()), dtype=torch.int32, device=device).reshape(spec.shape)
        elif spec.init == "ones":
            t = torch.ones(spec.shape, dtype=torch.float32, device=device)
            if norm_std:
                t += torch.randn(spec.shape, generator=g, dtype=torch.float32, device=device) * norm_std
        elif spec.init == "zeros":
            t = torch.zeros(spec.shape, dtype=torch.float32, device=device)
        else:
            t = torch.randn(spec.shape, generator=g, dtype=torch.float32, device=device) * std
        tensors[name] = t if spec.kind == "int" else t.to(storage_dtype(torch.bfloat16, spec.kind, dtype))
    model.load(tensors, dtype, device, pack_weights=pack_weights)
    return model
