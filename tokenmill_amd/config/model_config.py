"""Typed model configuration read from the architecture's own config.json keys.

Keys, fall-backs and the order in which end-of-sequence ids are collected follow the reference's
ModelConfig.from_pretrained_dir (reference src/infer/config.py:41-69).  Nothing here carries a
model size: a key without a fall-back in the reference is required.
"""
from __future__ import annotations

import json
from dataclasses import dataclass, field
from pathlib import Path


class ConfigError(ValueError):
    """config.json is missing a key, or holds a value the engine cannot run."""


def _require(raw: dict, key: str):
    if key not in raw or raw[key] is None:
        raise ConfigError(f"config.json has no '{key}'")
    return raw[key]


def collect_eos_ids(sources: list[dict]) -> tuple[int, ...]:
    """Ordered union of ``eos_token_id`` (int or list) over the given dicts
    (reference src/infer/config.py:45-53: generation_config.json first, then config.json)."""
    eos: list[int] = []
    for source in sources:
        val = source.get("eos_token_id")
        if val is None:
            continue
        for tok in val if isinstance(val, list) else [val]:
            if int(tok) not in eos:
                eos.append(int(tok))
    return tuple(eos)


@dataclass(frozen=True)
class Qwen2Config:
    """The Qwen2 / Qwen2.5 dense decoder (reference src/infer/config.py:13-39)."""

    vocab_size: int
    hidden_size: int
    intermediate_size: int
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    max_position_embeddings: int
    rope_theta: float
    rms_norm_eps: float
    tie_word_embeddings: bool
    eos_token_ids: tuple[int, ...] = field(default_factory=tuple)

    architecture = "Qwen2ForCausalLM"

    @property
    def num_kv_groups(self) -> int:
        return self.num_attention_heads // self.num_key_value_heads

    @property
    def q_size(self) -> int:
        return self.num_attention_heads * self.head_dim

    @property
    def kv_size(self) -> int:
        return self.num_key_value_heads * self.head_dim

    @classmethod
    def from_dict(cls, raw: dict, generation: dict | None = None) -> "Qwen2Config":
        heads = int(_require(raw, "num_attention_heads"))
        hidden = int(_require(raw, "hidden_size"))
        rope_theta = raw.get("rope_theta")
        if rope_theta is None:          # newer writers nest it (reference src/infer/config.py:54-56)
            rope_theta = (raw.get("rope_parameters") or {}).get("rope_theta", 10000.0)
        head_dim = raw.get("head_dim")
        if head_dim is None:            # derived when absent (reference src/infer/config.py:29-31)
            if hidden % heads:
                raise ConfigError(f"hidden_size {hidden} is not a multiple of num_attention_heads {heads}")
            head_dim = hidden // heads
        cfg = cls(
            vocab_size=int(_require(raw, "vocab_size")),
            hidden_size=hidden,
            intermediate_size=int(_require(raw, "intermediate_size")),
            num_hidden_layers=int(_require(raw, "num_hidden_layers")),
            num_attention_heads=heads,
            num_key_value_heads=int(raw.get("num_key_value_heads") or heads),
            head_dim=int(head_dim),
            max_position_embeddings=int(raw.get("max_position_embeddings", 32768)),
            rope_theta=float(rope_theta),
            rms_norm_eps=float(raw.get("rms_norm_eps", 1e-6)),
            tie_word_embeddings=bool(raw.get("tie_word_embeddings", False)),
            eos_token_ids=collect_eos_ids(([generation] if generation else []) + [raw]),
        )
        cfg.validate(raw)
        return cfg

    def validate(self, raw: dict | None = None) -> None:
        for name in ("vocab_size", "hidden_size", "intermediate_size", "num_hidden_layers",
                     "num_attention_heads", "num_key_value_heads", "head_dim", "max_position_embeddings"):
            if getattr(self, name) <= 0:
                raise ConfigError(f"{name} must be positive, got {getattr(self, name)}")
        if self.num_attention_heads % self.num_key_value_heads:
            raise ConfigError(f"num_attention_heads {self.num_attention_heads} is not a multiple of "
                              f"num_key_value_heads {self.num_key_value_heads}")
        if self.head_dim % 2:
            raise ConfigError(f"head_dim {self.head_dim} must be even for rotary pairs")
        if not self.rms_norm_eps > 0 or not self.rope_theta > 0:
            raise ConfigError("rms_norm_eps and rope_theta must be positive")
        raw = raw or {}
        # The reference's model keeps every key and knows one activation and one rotary table;
        # a checkpoint that asks for something else must not run silently as if it did not.
        if raw.get("use_sliding_window"):
            raise ConfigError("use_sliding_window=true is not supported by the Qwen2 model of this engine")
        if raw.get("hidden_act", "silu") != "silu":
            raise ConfigError(f"hidden_act '{raw.get('hidden_act')}' is not supported (silu only)")
        if raw.get("rope_scaling") not in (None, {}):
            raise ConfigError("rope_scaling is not supported")

    def to_json_dict(self) -> dict:
        """config.json contents that read back to this configuration."""
        d = {
            "architectures": [self.architecture],
            "model_type": "qwen2",
            "vocab_size": self.vocab_size,
            "hidden_size": self.hidden_size,
            "intermediate_size": self.intermediate_size,
            "num_hidden_layers": self.num_hidden_layers,
            "num_attention_heads": self.num_attention_heads,
            "num_key_value_heads": self.num_key_value_heads,
            "head_dim": self.head_dim,
            "max_position_embeddings": self.max_position_embeddings,
            "rope_theta": self.rope_theta,
            "rms_norm_eps": self.rms_norm_eps,
            "tie_word_embeddings": self.tie_word_embeddings,
            "hidden_act": "silu",
            "use_sliding_window": False,
        }
        if self.eos_token_ids:
            d["eos_token_id"] = list(self.eos_token_ids)
        return d


def read_json(path: Path) -> dict:
    try:
        return json.loads(path.read_text())
    except FileNotFoundError:
        raise ConfigError(f"{path} does not exist") from None
