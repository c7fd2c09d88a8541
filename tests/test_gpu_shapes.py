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
            assert_logits_close(row, plain.logits(ids[rid], dt)[p], dt, f"{name} shape {dtype_name} {rid} position {p}",
                                plain.bf16_noise((40, 25)) if dt == torch.bfloat16 else None)
        assert not session.manager.live
        del session
        torch.cuda.empty_cache()


LAYERS = {
    "0.5B": qwen2_config(num_hidden_layers=2, hidden_size=896, num_attention_heads=14, num_key_value_heads=2,
                         intermediate_size=4864, vocab_size=1000, rope_theta=1e6, rms_norm_eps=1e-6,
                         tie_word_embeddings=True),
    "7B": qwen2_config(num_hidden_layers=2, hidden_size=3584, num_attention_heads=28, num_key_value_heads=4,
                       intermediate_size=18944, vocab_size=1000, rope_theta=1e6, rms_norm_eps=1e-6,
                       tie_word_embeddings=False),
}


@pytest.fixture(scope="module")
def layer_models(tmp_path_factory):
    from conftest import Plain
    from tokenmill_amd.weights import write_random_model
    made = {}

    def get(name):
        if name not in made:
            d = write_random_model(LAYERS[name], tmp_path_factory.mktemp(f"layers{name}"), seed=8, std=0.02, norm_std=0.1)
            made[name] = (d, Plain(d))
        return made[name]

    return get


@pytest.mark.parametrize("dtype_name", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["0.5B", "7B"])
def test_every_cut_at_the_layer_sizes_of_the_published_shapes(layer_models, monkeypatch, name, dtype_name):
    """Two layers of the 0.5B and of the 7B shape (small vocabulary), replayed whole, with the last 32 tokens
    one by one, in portions down to two tokens, and mixed with up to four live requests on so few pages that
    they are used again: the fast paths of the real sizes (head size 64 and 128, groups of 7, the products
    that start at the norm, and for steps of 17 to 48 rows the products that keep the input in LDS) under
    every way of cutting, against the plain implementation."""
    from tokenmill_amd.replay import ReplaySession
    from test_gpu_replay import assert_all_given_back, check, mixed, portions, prefill_then_decode, run_trace, whole

    d, plain = layer_models(name)
    dt = {"float32": torch.float32, "bfloat16": torch.bfloat16}[dtype_name]
    lengths = [70, 41, 100, 56, 33, 88, 120, 64]
    reqs = {f"r{i}": random_ids(n, 1000, 600 + i) for i, n in enumerate(lengths)}
    session = ReplaySession(d, dtype_name, 4 * 128)            # four live requests of at most 128 tokens: 32 pages
    assert sum(-(-n // 16) for n in lengths) > session.num_pages
    steps = mixed(reqs, seed=12, live=4, max_portion=14)
    sizes = [sum(len(e["tokens"]) for e in st["entries"]) for st in steps]
    assert any(17 <= n <= 48 for n in sizes) and any(n <= 16 for n in sizes)
    for what, trace in (("whole", whole(reqs)), ("prefill+decode", prefill_then_decode(reqs)),
                        ("portions", portions(reqs)), ("mixed", steps)):
        got = run_trace(session, trace)
        check(got, plain, reqs, dt, f"{name} layers, {dtype_name}, {what}")
        assert_all_given_back(session)
    took = session.runner.program.counters()
    if dtype_name == "bfloat16":
        assert took["qkv_from_norm"] > 0 and took["gate_up_from_norm"] > 0 and took["qkv_plain"] > 0
        assert took["qkv_panel"] > 0 or name == "7B"          # a width of 3,584 does not fit a block's LDS
    else:
        assert took["qkv_plain"] > 0 and took["qkv_from_norm"] == 0
    # the same mixed trace launched from the parts' own code: the same bits
    by_parts = ReplaySession(d, dtype_name, 4 * 128)
    by_parts.runner.program = None
    again = run_trace(by_parts, steps)
    for key, row in run_trace(session, steps).items():
        assert torch.equal(row, again[key]), f"{name} layers, {dtype_name}: {key}"
    del by_parts
    del session
    torch.cuda.empty_cache()
