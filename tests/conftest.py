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

# A head size and a group the published shapes have (64; seven query heads on one kv head), and weights wide
# enough that attention is peaked and the logits spread over several units: a wrong key or mask moves them far.
TINY_D = qwen2_config(num_hidden_layers=2, hidden_size=448, num_attention_heads=7, num_key_value_heads=1,
                      intermediate_size=600, vocab_size=500, rope_theta=1e6, rms_norm_eps=1e-6,
                      tie_word_embeddings=False, eos_token_id=2)

# (config, weight seed, std of matrices and biases, std of the norm weights around 1)
TINY = {"A": (TINY_A, 0, 0.02, 0.0), "B": (TINY_B, 1, 0.02, 0.1), "C": (TINY_C, 2, 0.08, 0.2),
        "D": (TINY_D, 3, 0.06, 0.1)}


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

    def bf16_noise(self, lengths=(96, 61, 30), orders=None) -> float:
        """How far the bfloat16 logits of this model move when only the order of the 32-bit sums changes:
        the largest difference, over a few random sequences, between the plain implementation's usual
        summation order and each of its other ones. Measured, per model, on the CPU; the bfloat16
        comparisons take their bound from it."""
        if "noise" not in self._cache:
            worst = 0.0
            for i, n in enumerate(lengths):
                ids = random_ids(n, self.cfg["vocab"], 9000 + i)
                a = self.logits(ids, torch.bfloat16)
                for k in range(1, orders or self.P.NUM_ORDERS):
                    with self.P.summation_order(k):
                        b = self.P.forward_logits(self.w, self.cfg, ids, torch.bfloat16)
                    worst = max(worst, float((a - b).abs().max()))
            self._cache["noise"] = worst
        return self._cache["noise"]


@pytest.fixture(scope="session")
def plains(model_dirs):
    return {name: Plain(d) for name, d in model_dirs.items()}


def random_ids(n: int, vocab: int, seed: int) -> list[int]:
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()
