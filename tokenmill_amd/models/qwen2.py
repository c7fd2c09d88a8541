"""Qwen2 / Qwen2.5 dense decoder assembled from parts (reference src/infer/model/qwen2.py:13-52,
src/infer/model/layers.py:127-164).

Every layer: RMSNorm -> grouped-query attention (q, k, v with bias, rotary positions over the whole
head, scale head_dim^-0.5, output projection without bias) -> RMSNorm -> SwiGLU without biases.
Tensor names are the checkpoint's (reference src/infer/model/loader.py:98-119).
"""
from __future__ import annotations

from tokenmill_amd.config.model_config import Qwen2Config
from tokenmill_amd.config.registry import register_architecture
from tokenmill_amd.models.decoder import DecoderModel
from tokenmill_amd.parts import GQAttention, OutputHead, PreNormBlock, RMSNorm, RotaryEmbedding, SwiGLU, TokenEmbedding


def build_qwen2(cfg: Qwen2Config, max_positions: int | None = None) -> DecoderModel:
    n_pos = min(max_positions or cfg.max_position_embeddings, cfg.max_position_embeddings)
    rope = RotaryEmbedding(cfg.head_dim, cfg.rope_theta, n_pos)          # one table for all layers
    embedding = TokenEmbedding(cfg.vocab_size, cfg.hidden_size)
    layers = []
    for _ in range(cfg.num_hidden_layers):
        attn = GQAttention(cfg.hidden_size, cfg.num_attention_heads, cfg.num_key_value_heads, cfg.head_dim,
                           scale=cfg.head_dim ** -0.5, position=rope, qkv_bias=True, o_bias=False, window=None)
        mlp = SwiGLU(cfg.hidden_size, cfg.intermediate_size, bias=False)
        layers.append(PreNormBlock(RMSNorm(cfg.hidden_size, cfg.rms_norm_eps), attn,
                                   RMSNorm(cfg.hidden_size, cfg.rms_norm_eps), mlp))
    head = OutputHead(cfg.hidden_size, cfg.vocab_size, tied_to=embedding if cfg.tie_word_embeddings else None)
    ignorable = ("*rotary_emb*",) + (("lm_head.weight",) if cfg.tie_word_embeddings else ())
    return DecoderModel(cfg, embedding, layers, RMSNorm(cfg.hidden_size, cfg.rms_norm_eps), head, ignorable=ignorable)


register_architecture(Qwen2Config.architecture, Qwen2Config.from_dict, build_qwen2, replace=True)
