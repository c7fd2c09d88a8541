"""The layer sizes of the Qwen2.5 0.5B / 7B / 32B shapes (head size 64 and 128, groups of 7 and 5,
widths 896 / 3584 / 5120, which take the kernels' other code paths), each with few layers and, for the
two large ones, a small vocabulary so that the plain implementation on the CPU stays quick."""
from __future__ import annotations

import pytest
import torch

from conftest import qwen2_config, random_ids
from tolerances import assert_logits_close

pytestmark = pytest.mark.gpu

SHAPES = {
    "0.5B": qwen2_config(num_hidden_layers=2, hidden_size=896, num_attention_heads=14, num_key_value_heads=2,
                         intermediate_size=4864, vocab_size=151936, rope_theta=1e6, rms_norm_eps=1e-6,
                         tie_word_embeddings=True),
    "7B": qwen2_config(num_hidden_layers=1, hidden_size=3584, num_attention_heads=28, num_key_value_heads=4,
                       intermediate_size=18944, vocab_size=2048, rope_theta=1e6, rms_norm_eps=1e-6,
                       tie_word_embeddings=False),
    "32B": qwen2_config(num_hidden_layers=1, hidden_size=5120, num_attention_heads=40, num_key_value_heads=8,
                        intermediate_size=27648, vocab_size=2048, rope_theta=1e6, rms_norm_eps=1e-6,
                        tie_word_embeddings=False),
}


@pytest.mark.parametrize("name,dtypes", [("0.5B", ("float32", "bfloat16")), ("7B", ("bfloat16",)), ("32B", ("bfloat16",))])
def test_layer_sizes_of_the_published_shapes(tmp_path, name, dtypes):
    from conftest import Plain
    from tokenmill_amd.replay import ReplaySession
    from tokenmill_amd.weights import write_random_model
    from test_gpu_replay import run_trace

    cfg = SHAPES[name]
    d = write_random_model(cfg, tmp_path / name, seed=7, std=0.02, norm_std=0.1)
    plain = Plain(d)
    ids = {"a": random_ids(70, cfg["vocab_size"], 1), "b": random_ids(21, cfg["vocab_size"], 2)}
    steps = [
        {"step": 0, "entries": [{"id": "a", "tokens": ids["a"][:50], "want": [0, 17, 49]}], "end": []},
        {"step": 1, "entries": [{"id": "a", "tokens": ids["a"][50:60], "want": [9]},
                                {"id": "b", "tokens": ids["b"][:20], "want": [19]}], "end": []},
    ] + [{"step": 2 + i, "entries": [{"id": "a", "tokens": [ids["a"][60 + i]], "want": [0]}] +
          ([{"id": "b", "tokens": [ids["b"][20]], "want": [0]}] if i == 0 else []), "end": ["b"] if i == 0 else []}
         for i in range(10)]
    steps[-1]["end"] = ["a"]
    for dtype_name in dtypes:
        dt = {"float32": torch.float32, "bfloat16": torch.bfloat16}[dtype_name]
        session = ReplaySession(d, dtype_name, 256)
        got = run_trace(session, steps)
        assert len(got) == 3 + 2 + 10 + 1
        for (rid, p), row in got.items():
            assert_logits_close(row, plain.logits(ids[rid], dt)[p], dt, f"{name} shape {dtype_name} {rid} position {p}")
        assert not session.manager.live
        del session
        torch.cuda.empty_cache()
