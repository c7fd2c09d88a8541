"""Shared fixtures: tiny configurations, model folders with random weights, the plain implementation."""
from __future__ import annotations

import sys
from pathlib import Path

import pytest
import torch

ROOT = Path(__file__).resolve().parent.parent
sys.path.insert(0, str(ROOT))
sys.path.insert(0, str(Path(__file__).resolve().parent))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X (run on the GPU box)")


def qwen2_config(**kw) -> dict:
    base = {"architectures": ["Qwen2ForCausalLM"], "model_type": "qwen2", "hidden_act": "silu",
            "max_position_embeddings": 4096, "use_sliding_window": False}
    base.update(kw)
    return base


# Two tiny configurations that differ in every size and option (and a third with sizes that are
# no powers of two and a head size given apart from hidden / heads).
TINY_A = qwen2_config(num_hidden_layers=2, hidden_size=64, num_attention_heads=4, num_key_value_heads=2,
                      intermediate_size=128, vocab_size=256, rope_theta=10000.0, rms_norm_eps=1e-6,
                      tie_word_embeddings=True, eos_token_id=[3, 5])
TINY_B = qwen2_config(num_hidden_layers=3, hidden_size=192, num_attention_heads=6, num_key_value_heads=1,
                      intermediate_size=320, vocab_size=384, rope_theta=1e6, rms_norm_eps=1e-5,
                      tie_word_embeddings=False, eos_token_id=7)
TINY_C = qwen2_config(num_hidden_layers=2, hidden_size=120, num_attention_heads=6, num_key_value_heads=3,
                      head_dim=48, intermediate_size=200, vocab_size=307, rope_theta=50000.0, rms_norm_eps=3e-6,
                      tie_word_embeddings=False)

# (config, weight seed, std of matrices and biases, std of the norm weights around 1)
TINY = {"A": (TINY_A, 0, 0.02, 0.0), "B": (TINY_B, 1, 0.02, 0.1), "C": (TINY_C, 2, 0.08, 0.2)}


@pytest.fixture(scope="session")
def model_dirs(tmp_path_factory):
    """name -> folder with config.json and model.safetensors (random weights, bfloat16 storage)."""
    from tokenmill_amd.weights.random_init import write_random_model

    out = {}
    for name, (cfg, seed, std, norm_std) in TINY.items():
        d = tmp_path_factory.mktemp(f"tiny{name}")
        write_random_model(cfg, d, seed=seed, std=std, norm_std=norm_std)
        out[name] = d
    return out


class Plain:
    """The plain implementation's view of a model folder."""

    def __init__(self, model_dir):
        from plain import qwen2_plain as P

        self.P = P
        self.cfg = P.read_config(model_dir)
        self.w = P.read_weights(model_dir)
        self._cache: dict = {}

    def logits(self, ids, dt=torch.float32):
        key = (tuple(ids), dt)
        if key not in self._cache:
            self._cache[key] = self.P.forward_logits(self.w, self.cfg, list(ids), dt)
        return self._cache[key]


@pytest.fixture(scope="session")
def plains(model_dirs):
    return {name: Plain(d) for name, d in model_dirs.items()}


def random_ids(n: int, vocab: int, seed: int) -> list[int]:
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()
