"""Configurations of the architecture with the head sizes, groups and page sizes that neither the tiny
configurations nor the published shapes have (head sizes 80, 96 and 112, groups of 1, 4 and 8, a head size
given apart from hidden / heads, pages of 32 and 64, widths and feed-forward sizes that are no multiples of 8, 4
or 2), each through every way of cutting the work, in both
precisions, against the plain implementation: the kernels take every size the configuration allows, or
another kernel does."""
from __future__ import annotations

import pytest
import torch

from conftest import qwen2_config, random_ids

pytestmark = pytest.mark.gpu

OTHER = {
    "d80-g8": (qwen2_config(num_hidden_layers=2, hidden_size=1280, num_attention_heads=16, num_key_value_heads=2,
                            intermediate_size=1000, vocab_size=307, rope_theta=1e4, rms_norm_eps=1e-5,
                            tie_word_embeddings=True), 16, 0.03),
    "d112-g4": (qwen2_config(num_hidden_layers=1, hidden_size=328, num_attention_heads=4, num_key_value_heads=1,
                             head_dim=112, intermediate_size=616, vocab_size=1000, rope_theta=5e4, rms_norm_eps=1e-6,
                             tie_word_embeddings=False), 32, 0.05),
    "d96-g1": (qwen2_config(num_hidden_layers=3, hidden_size=288, num_attention_heads=3, num_key_value_heads=3,
                            intermediate_size=360, vocab_size=1000, rope_theta=1e6, rms_norm_eps=3e-6,
                            tie_word_embeddings=False), 16, 0.02),
    # widths, feed-forward sizes and vocabularies that are no multiples of 8, of 4 or of 2: the products that need
    # aligned rows give way to the ones that do not
    "odd-36": (qwen2_config(num_hidden_layers=2, hidden_size=36, num_attention_heads=2, num_key_value_heads=1, head_dim=16,
                            intermediate_size=37, vocab_size=97, rope_theta=1e4, rms_norm_eps=1e-6,
                            tie_word_embeddings=False), 16, 0.05),
    "odd-250": (qwen2_config(num_hidden_layers=2, hidden_size=250, num_attention_heads=5, num_key_value_heads=1,
                             head_dim=48, intermediate_size=333, vocab_size=501, rope_theta=1e4, rms_norm_eps=1e-6,
                             tie_word_embeddings=True), 8, 0.05),
    "d16-g8": (qwen2_config(num_hidden_layers=3, hidden_size=256, num_attention_heads=16, num_key_value_heads=2,
                            intermediate_size=360, vocab_size=250, rope_theta=1e4, rms_norm_eps=1e-6,
                            tie_word_embeddings=True), 64, 0.05),
}


@pytest.mark.parametrize("dtype_name", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", sorted(OTHER))
def test_every_cut_at_other_head_sizes_groups_and_pages(tmp_path_factory, name, dtype_name):
    from conftest import Plain
    from tokenmill_amd.replay import ReplaySession
    from tokenmill_amd.weights import write_random_model
    from test_gpu_replay import assert_all_given_back, check, mixed, portions, prefill_then_decode, run_trace, whole

    cfg, page, std = OTHER[name]
    d = write_random_model(cfg, tmp_path_factory.mktemp(name), seed=31, std=std, norm_std=0.1)
    plain = Plain(d)
    dt = {"float32": torch.float32, "bfloat16": torch.bfloat16}[dtype_name]
    reqs = {f"r{j}": random_ids(n, cfg["vocab_size"], 700 + j) for j, n in enumerate((3, 41, 70, 17, 88, 56))}
    session = ReplaySession(d, dtype_name, 4 * 128, page_size=page)
    for what, trace in (("whole", whole(reqs)), ("prefill+decode", prefill_then_decode(reqs)),
                        ("portions", portions(reqs)), ("mixed", mixed(reqs, seed=5, live=4, max_portion=19))):
        got = run_trace(session, trace)
        check(got, plain, reqs, dt, f"{name}, {dtype_name}, {what}")
        assert_all_given_back(session)
