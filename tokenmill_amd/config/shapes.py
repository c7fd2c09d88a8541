"""Named configurations shipped with the package as config.json files (`shapes/*.json`): the published
Qwen2.5 sizes this engine is measured at and two tiny ones. They are data, read like any config.json."""
from __future__ import annotations

import json
from pathlib import Path

_DIR = Path(__file__).parent / "shapes"
_ALIASES = {"0.5b": "qwen2.5-0.5b", "7b": "qwen2.5-7b", "32b": "qwen2.5-32b", "tinya": "tiny-a", "tinyb": "tiny-b"}


def shape_names() -> list[str]:
    return sorted(p.stem for p in _DIR.glob("*.json"))


def read_shape(name_or_path: str) -> dict:
    """config.json contents for a shipped name ("qwen2.5-7b", "7b", "tiny-a", ...), a config.json file, or a
    folder holding one."""
    key = name_or_path.lower()
    key = _ALIASES.get(key, key)
    shipped = _DIR / f"{key}.json"
    if shipped.is_file():
        return json.loads(shipped.read_text())
    path = Path(name_or_path)
    if path.is_dir():
        path = path / "config.json"
    if not path.is_file():
        raise FileNotFoundError(f"{name_or_path!r} is neither a config.json (or its folder) nor one of the shipped "
                                f"shapes: {', '.join(shape_names())}")
    return json.loads(path.read_text())
