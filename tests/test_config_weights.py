"""Configuration, registry and weight loading (CPU)."""
from __future__ import annotations

import json

import pytest
import torch
from safetensors.torch import load_file, save_file

from conftest import TINY_A, TINY_B, TINY_C, qwen2_config
from tokenmill_amd.config import ConfigError, Qwen2Config, get_architecture, known_architectures, load_config
from tokenmill_amd.config.engine_config import EngineConfig, add_engine_args, engine_config_from_args
from tokenmill_amd.weights import TensorSpec, WeightsError, read_checkpoint, write_random_model


def test_config_reads_its_own_keys_and_derives_the_rest():
    cfg = Qwen2Config.from_dict(TINY_A)
    assert (cfg.num_hidden_layers, cfg.hidden_size, cfg.num_attention_heads, cfg.num_key_value_heads) == (2, 64, 4, 2)
    assert cfg.head_dim == 16 and cfg.num_kv_groups == 2 and cfg.q_size == 64 and cfg.kv_size == 32
    assert cfg.tie_word_embeddings and cfg.rope_theta == 10000.0 and cfg.eos_token_ids == (3, 5)
    c = Qwen2Config.from_dict(TINY_C)
    assert c.head_dim == 48 and c.q_size == 288 != c.hidden_size       # a head size given apart from hidden / heads


def test_config_fallbacks_are_the_references():
    """reference src/infer/config.py:54-67"""
    raw = {k: v for k, v in TINY_B.items() if k not in ("num_key_value_heads", "rope_theta", "rms_norm_eps",
                                                         "tie_word_embeddings", "max_position_embeddings")}
    cfg = Qwen2Config.from_dict(raw)
    assert cfg.num_key_value_heads == cfg.num_attention_heads
    assert cfg.rope_theta == 10000.0 and cfg.rms_norm_eps == 1e-6 and cfg.max_position_embeddings == 32768
    assert cfg.tie_word_embeddings is False
    assert Qwen2Config.from_dict(dict(raw, rope_parameters={"rope_theta": 5e5})).rope_theta == 5e5


def test_eos_ids_come_from_generation_config_first():
    """reference src/infer/config.py:45-53"""
    cfg = Qwen2Config.from_dict(dict(TINY_A, eos_token_id=[3, 5]), {"eos_token_id": [9, 3]})
    assert cfg.eos_token_ids == (9, 3, 5)


@pytest.mark.parametrize("bad, word", [
    ({"hidden_size": None}, "hidden_size"), ({"num_key_value_heads": 3}, "multiple"),
    ({"use_sliding_window": True}, "sliding"), ({"hidden_act": "gelu"}, "hidden_act"),
    ({"rope_scaling": {"type": "yarn"}}, "rope_scaling"), ({"hidden_size": 66}, "multiple"),
    ({"vocab_size": 0}, "positive")])
def test_config_refuses_what_it_cannot_run(bad, word):
    with pytest.raises(ConfigError, match=word):
        Qwen2Config.from_dict(dict(TINY_A, **bad))


def test_a_context_or_head_size_the_model_cannot_run_is_refused_where_the_model_is_built():
    """Not by the first step that reaches a kernel: the reference sizes its rotary table from
    min(max_model_len, max_position_embeddings) at load (reference src/infer/model/qwen2.py:34)."""
    from tokenmill_amd.engine.loading import check_positions
    from tokenmill_amd.models.qwen2 import build_qwen2
    cfg = Qwen2Config.from_dict(dict(TINY_A, max_position_embeddings=512))
    check_positions(cfg, 512)
    check_positions(cfg, None)
    with pytest.raises(ConfigError, match="max_position_embeddings 512"):
        check_positions(cfg, 513)
    with pytest.raises(ConfigError, match="at least 1"):
        check_positions(cfg, 0)
    assert build_qwen2(cfg, 128).layers[0].mixer.position.max_positions == 128
    # head sizes: even for the rotary pairs (the configuration's own rule), a multiple of 4 up to 256 for the kernels
    for head_dim, hidden in ((6, 24), (260, 1040)):
        bad = Qwen2Config.from_dict(dict(TINY_A, hidden_size=hidden, head_dim=head_dim))
        with pytest.raises(ValueError, match=f"head size {head_dim}"):
            build_qwen2(bad, 128)
    build_qwen2(Qwen2Config.from_dict(dict(TINY_A, head_dim=20)), 128)


def test_registry_chooses_by_config_json(tmp_path):
    assert "Qwen2ForCausalLM" in known_architectures()
    (tmp_path / "config.json").write_text(json.dumps(TINY_B))
    arch, cfg = load_config(tmp_path)
    assert arch.name == "Qwen2ForCausalLM" and isinstance(cfg, Qwen2Config) and cfg.hidden_size == 192
    (tmp_path / "config.json").write_text(json.dumps(dict(TINY_B, architectures=["NopeForCausalLM"])))
    with pytest.raises(ConfigError, match="Qwen2ForCausalLM"):           # the error lists what is known
        load_config(tmp_path)
    with pytest.raises(ConfigError, match="architectures"):
        get_architecture  # noqa: B018
        (tmp_path / "config.json").write_text(json.dumps({k: v for k, v in TINY_B.items() if k != "architectures"}))
        load_config(tmp_path)


def test_config_round_trips_through_json():
    cfg = Qwen2Config.from_dict(TINY_C)
    assert Qwen2Config.from_dict(cfg.to_json_dict()) == cfg


def test_engine_flags_mirror_the_fields():
    import argparse
    p = add_engine_args(argparse.ArgumentParser())
    a = p.parse_args(["--model", "m", "--block-size", "8", "--max-batched-tokens", "12", "--enable-chunked-prefill",
                      "--kv-cache-mb", "4", "--watermark", "0.05", "--dtype", "float32"])
    cfg = engine_config_from_args(a)
    assert (cfg.model, cfg.block_size, cfg.max_num_batched_tokens, cfg.enable_chunked_prefill) == ("m", 8, 12, True)
    assert cfg.kv_cache_mb == 4 and cfg.watermark == 0.05 and cfg.dtype == "float32"
    assert p.parse_args(["--max-num-batched-tokens", "7"]).max_num_batched_tokens == 7
    d = EngineConfig()
    assert (d.block_size, d.max_model_len, d.max_num_seqs, d.max_num_batched_tokens, d.watermark, d.policy,
            d.max_waiting_steps, d.gpu_memory_utilization, d.seed) == (16, 2048, 128, 2048, 0.01, "prefill_first",
                                                                       20, 0.90, 0)     # reference config.py:72-107


# ----------------------------------------------------------------------------------------------- weights

def _specs(cfg_dict):
    arch = get_architecture("Qwen2ForCausalLM")
    model = arch.build_model(arch.config_from_dict(cfg_dict, None))
    return model, model.tensor_specs()


def test_random_model_folder_reads_back_by_name(tmp_path):
    d = write_random_model(TINY_B, tmp_path / "m", seed=1, std=0.02, norm_std=0.1)
    assert (d / "config.json").exists() and (d / "model.safetensors").exists()
    model, specs = _specs(TINY_B)
    assert "lm_head.weight" in specs and "model.layers.2.self_attn.k_proj.bias" in specs
    t = read_checkpoint(d, specs, torch.bfloat16, "cpu", model.ignorable)
    assert set(t) == set(specs)
    assert all(v.dtype == torch.bfloat16 for v in t.values())
    assert t["model.layers.0.self_attn.q_proj.weight"].shape == (192, 192)
    w = t["model.layers.1.mlp.gate_proj.weight"].float()
    assert abs(w.std().item() - 0.02) < 0.002 and abs(w.mean().item()) < 0.001
    n = t["model.layers.1.input_layernorm.weight"].float()
    assert abs(n.mean().item() - 1) < 0.05 and 0.05 < n.std().item() < 0.15
    again = write_random_model(TINY_B, tmp_path / "m2", seed=1, std=0.02, norm_std=0.1)
    a, b = load_file(d / "model.safetensors"), load_file(again / "model.safetensors")
    assert all(torch.equal(a[k], b[k]) for k in a)                      # the seed fixes every tensor
    other = load_file(write_random_model(TINY_B, tmp_path / "m3", seed=2) / "model.safetensors")
    assert not torch.equal(a["lm_head.weight"], other["lm_head.weight"])
    t32 = read_checkpoint(d, specs, torch.float32, "cpu", model.ignorable)
    assert all(v.dtype == torch.float32 for v in t32.values())
    assert torch.equal(t32["lm_head.weight"], t["lm_head.weight"].float())


def test_tied_model_has_no_second_matrix_and_ignores_one_in_the_file(tmp_path):
    d = write_random_model(TINY_A, tmp_path / "m", seed=0)
    model, specs = _specs(TINY_A)
    assert "lm_head.weight" not in specs
    tensors = load_file(d / "model.safetensors")
    tensors["lm_head.weight"] = tensors["model.embed_tokens.weight"].clone()
    tensors["model.layers.0.self_attn.rotary_emb.inv_freq"] = torch.zeros(8)
    save_file(tensors, d / "model.safetensors")
    read_checkpoint(d, specs, torch.bfloat16, "cpu", model.ignorable)   # skipped as the reference skips them


def test_one_error_lists_missing_unexpected_and_wrong_shapes(tmp_path):
    d = write_random_model(TINY_B, tmp_path / "m", seed=1)
    model, specs = _specs(TINY_B)
    tensors = load_file(d / "model.safetensors")
    del tensors["model.layers.1.self_attn.q_proj.bias"]
    del tensors["lm_head.weight"]
    tensors["model.layers.0.mlp.extra_proj.weight"] = torch.zeros(3, 3)
    tensors["model.norm.weight"] = torch.ones(191)
    tensors["model.layers.2.mlp.down_proj.weight"] = torch.zeros(320, 192)      # transposed
    save_file(tensors, d / "model.safetensors")
    with pytest.raises(WeightsError) as e:
        read_checkpoint(d, specs, torch.bfloat16, "cpu", model.ignorable)
    err = e.value
    assert err.missing == ["lm_head.weight", "model.layers.1.self_attn.q_proj.bias"]
    assert err.unexpected == ["model.layers.0.mlp.extra_proj.weight"]
    assert [n for n, _, _ in err.wrong_shape] == ["model.layers.2.mlp.down_proj.weight", "model.norm.weight"]
    msg = str(err)
    for word in ("missing", "unexpected", "wrong shapes", "lm_head.weight", "extra_proj", "[191]", "[192]"):
        assert word in msg


def test_no_safetensors_files_is_an_error(tmp_path):
    (tmp_path / "config.json").write_text(json.dumps(TINY_A))
    with pytest.raises(WeightsError, match="no .safetensors files"):
        read_checkpoint(tmp_path, {}, torch.bfloat16, "cpu")


def test_a_tensor_stored_in_32_bit_stays_so_and_integer_tables_become_int32(tmp_path):
    save_file({"a": torch.randn(4, 4), "b": torch.randn(4).bfloat16(), "c": torch.randn(4).half(),
               "t": torch.arange(6, dtype=torch.int64)}, tmp_path / "model.safetensors")
    specs = {"a": TensorSpec((4, 4)), "b": TensorSpec((4,)), "c": TensorSpec((4,)), "t": TensorSpec((6,), kind="int")}
    t = read_checkpoint(tmp_path, specs, torch.bfloat16, "cpu")
    assert t["a"].dtype == torch.float32 and t["b"].dtype == torch.bfloat16 and t["c"].dtype == torch.bfloat16
    assert t["t"].dtype == torch.int32
    t = read_checkpoint(tmp_path, specs, torch.float32, "cpu")
    assert {t[k].dtype for k in "abc"} == {torch.float32} and t["t"].dtype == torch.int32
    with pytest.raises(WeightsError, match="integer"):
        read_checkpoint(tmp_path, dict(specs, a=TensorSpec((4, 4), kind="int")), torch.bfloat16, "cpu")


def test_shipped_shapes_read_by_name_alias_or_path(tmp_path):
    from tokenmill_amd.config.shapes import read_shape, shape_names

    assert {"qwen2.5-0.5b", "qwen2.5-7b", "qwen2.5-32b", "tiny-a", "tiny-b"} <= set(shape_names())
    for name in shape_names():
        raw = read_shape(name)
        cfg = get_architecture(raw["architectures"][0]).config_from_dict(raw, None)
        assert cfg.num_attention_heads % cfg.num_key_value_heads == 0
    assert read_shape("7B") == read_shape("qwen2.5-7b")
    assert read_shape("0.5b")["hidden_size"] == 896 and read_shape("0.5b")["tie_word_embeddings"] is True
    (tmp_path / "config.json").write_text(json.dumps(qwen2_config(**TINY_B)))
    assert read_shape(str(tmp_path)) == read_shape(str(tmp_path / "config.json")) == qwen2_config(**TINY_B)
    with pytest.raises(FileNotFoundError, match="shipped shapes"):
        read_shape("no-such-shape")
