"""One registry from an architecture's name (config.json ``architectures[0]``) to its model.

The reference constructs its only model class directly (reference src/infer/model/loader.py:18,55);
here the name in config.json chooses a configuration class and a function that assembles the
model from parts, so another architecture is one more ``register_architecture`` call.
"""
from __future__ import annotations

from dataclasses import dataclass
from pathlib import Path
from typing import Any, Callable

from tokenmill_amd.config.model_config import ConfigError, read_json


@dataclass(frozen=True)
class Architecture:
    name: str
    config_from_dict: Callable[[dict, dict | None], Any]    # (config.json, generation_config.json) -> typed config
    build_model: Callable[..., Any]                         # (config, dtype, device, max_positions) -> ModelSpec


_REGISTRY: dict[str, Architecture] = {}


def register_architecture(name: str, config_from_dict, build_model, replace: bool = False) -> Architecture:
    if name in _REGISTRY and not replace:
        raise ValueError(f"architecture '{name}' is already registered")
    arch = Architecture(name, config_from_dict, build_model)
    _REGISTRY[name] = arch
    return arch


def known_architectures() -> list[str]:
    _ensure_builtin()
    return sorted(_REGISTRY)


def get_architecture(name: str) -> Architecture:
    _ensure_builtin()
    if name not in _REGISTRY:
        raise ConfigError(f"unknown architecture '{name}'; known: {sorted(_REGISTRY)}")
    return _REGISTRY[name]


def architecture_name(raw: dict) -> str:
    archs = raw.get("architectures")
    if not archs or not isinstance(archs, list):
        raise ConfigError("config.json has no 'architectures' list to choose the model by")
    return str(archs[0])


def load_config(model_dir: str | Path):
    """(Architecture, typed config) for a model folder."""
    model_dir = Path(model_dir)
    raw = read_json(model_dir / "config.json")
    gen_path = model_dir / "generation_config.json"
    generation = read_json(gen_path) if gen_path.exists() else None
    arch = get_architecture(architecture_name(raw))
    return arch, arch.config_from_dict(raw, generation)


def _ensure_builtin() -> None:
    # importing the package's models registers them
    import tokenmill_amd.models  # noqa: F401
