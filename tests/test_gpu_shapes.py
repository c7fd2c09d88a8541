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
    "32B": qwen2_config(num_hidden_layers=1, hidden_size=5120, num_attention_heads=40, num_key_value_heads=8,
                        intermediate_size=27648, vocab_size=1000, rope_theta=1e6, rms_norm_eps=1e-6,
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
@pytest.mark.parametrize("name", ["0.5B", "7B", "32B"])
def test_every_cut_at_the_layer_sizes_of_the_published_shapes(layer_models, monkeypatch, name, dtype_name):
    """Two layers of the 0.5B and of the 7B shape and one of the 32B shape (small vocabulary; a width of 5,120, a
    group of 5, a feed-forward of 27,648), replayed whole, with the last 32 tokens
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
        assert took["qkv_plain"] > 0
        if name == "32B":       # at this width the products that stream the matrix through windows of K take every step of up to 64 rows
            assert took["qkv_from_norm"] == 0 and took["gate_up_from_norm"] == 0
            assert took["qkv_stream"] > 0 and took["gate_up_stream"] > 0
        else:
            assert took["qkv_from_norm"] > 0 and took["gate_up_from_norm"] > 0
        assert took["qkv_panel"] > 0 or name != "0.5B"        # widths of 3,584 and 5,120 do not fit a block's LDS
    else:
        assert took["qkv_plain"] > 0 and took["qkv_from_norm"] == 0
    del session
    torch.cuda.empty_cache()


def _long_prompts(n_requests: int, seed: int) -> list[list[int]]:
    """Prompts of 2,100 to 2,303 ids; every fourth so close below 2,304 = 9 * 256 keys that its decode steps
    cross that edge of the split attention's 256-key chunks."""
    lengths = [2100 + (37 * i) % 200 if i % 4 else 2303 - (i // 4) % 12 for i in range(n_requests)]
    return [random_ids(n, 1000, seed + i) for i, n in enumerate(lengths)]


@pytest.mark.parametrize("name,n_requests,n_checked", [("0.5B", 8, 8), ("0.5B", 40, 6), ("7B", 8, 2), ("7B", 40, 3),
                                                       ("32B", 8, 2)])
def test_the_measured_configuration_against_the_plain_implementation(layer_models, name, n_requests, n_checked):
    """What the headline benchmark runs (reference tests/test_gpu.py:132-149 compares its graph path with its eager
    one at the real model): bfloat16 engines at the layer sizes of the 0.5B, 7B and 32B shapes with max_model_len 4,096,
    decode steps replayed from HIP graphs over contexts above 2,048 keys (the split attention inside the graph at
    8 requests, the one-block attention and the 48-row bucket's products at 40), once with the library's
    algorithms chosen by timing and the prompts cut into portions. Tokens are checked against the plain
    implementation (for some requests: it takes seconds a sequence at these widths)."""
    from test_gpu_engine import make_engine, verify
    from tokenmill_amd import SamplingParams

    d, plain = layer_models(name)
    prompts = _long_prompts(n_requests, 4000)
    sp = SamplingParams(max_tokens=16, ignore_eos=True)
    common = dict(block_size=16, kv_cache_mb=None, num_blocks=n_requests * 146 + 8, max_model_len=4096,
                  max_num_seqs=64, max_num_batched_tokens=4096)
    outs = {}
    for what, kw in (("eager", dict(hip_graphs=False)),
                     ("graphs", dict(hip_graphs=True)),
                     ("graphs, timed", dict(hip_graphs=True, tune_gemm=True)),
                     ("graphs, chunked", dict(hip_graphs=True, enable_chunked_prefill=True, max_num_batched_tokens=1024))):
        eng = make_engine(d, "bfloat16", **{**common, **kw})
        outs[what] = eng.generate(prompts, sp)
        if "chunked" in what:                     # the early requests decode beside the later ones' portions
            assert eng.stats["mixed_steps"] > 0 and eng.runner.step_graphs.replays > 0
        elif kw["hip_graphs"]:                    # every prompt first, then all requests decode together
            assert eng.runner.graphs.replays >= 14 and not eng.runner.graphs.failed, what
            assert (48 if n_requests == 40 else 8) in eng.runner.graphs.buckets
        eng.cache.check_invariants()
        assert eng.cache.num_free_pages == eng.cache.num_pages
        took = eng.runner.program.counters()
        if "chunked" not in what:                 # whole prompts of 2,100 and more tokens: the attention that shares a
            # tile's keys among the seven (five) heads of a kv head at head size 128, the one that splits them at 64
            assert (took["prefill_shared_keys"] > 0) == (name != "0.5B") and (took["prefill_split_keys"] > 0) == (name == "0.5B")
        del eng
        torch.cuda.empty_cache()
    # Up to 16 rows every kernel fixes its order of additions by the sizes alone: padding a step to its bucket
    # changes no bit. Beyond that the products are the library's, which may pick another algorithm for the 48
    # rows of a bucket than for the 40 of the eager step: then the logits agree up to rounding, and a token can
    # differ where two candidates are a near-tie (after which the two runs generate different sequences, each
    # of which must be right by itself). Such requests are a minority, and each is checked against the plain
    # implementation, beside a sample spread over the batch (the first is one that crosses 2,304 keys).
    if n_requests <= 16:
        assert outs["graphs"] == outs["eager"]
    checked = {(i * (n_requests - 1)) // max(n_checked - 1, 1) for i in range(n_checked)}
    for got in outs.values():
        differing = {i for i in range(n_requests) if got[i] != outs["eager"][i]}
        assert len(differing) <= max(1, n_requests // 4), f"{len(differing)} requests differ from the eager run"
        checked |= differing
    for what, got in outs.items():
        for i in sorted(checked):
            verify(plain, prompts[i], got[i], torch.bfloat16)
