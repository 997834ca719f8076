"""Qwen3 dense decoder from parts (src/models/qwen3.hpp): grouped-query attention with per-head
q/k RMS norm and half-split rotary positions, SwiGLU feed-forward, pre-RMS-norm blocks, an
output head that may be tied to the embedding.  Tensor names: src/models/qwen3.hpp:20-30, 44-46."""
from __future__ import annotations

from ..config.model_config import Qwen3Config
from ..config.registry import register_architecture
from ..parts import GatedMLP, LMHead, PagedAttention, PreNormBlock, RMSNorm, RotaryEmbedding, TokenEmbedding
from .base import DecoderModel


def build_qwen3(cfg: Qwen3Config) -> DecoderModel:
    embed = TokenEmbedding(cfg.vocab_size, cfg.hidden_size)
    rotary = RotaryEmbedding(cfg.head_dim, cfg.rope_theta)
    layers = []
    for _ in range(cfg.num_hidden_layers):
        attn = PagedAttention(cfg.hidden_size, cfg.num_attention_heads, cfg.num_key_value_heads, cfg.head_dim,
                              position=rotary, qk_norm_eps=cfg.rms_norm_eps)
        mlp = GatedMLP(cfg.hidden_size, cfg.intermediate_size, cfg.hidden_act)
        layers.append(PreNormBlock(RMSNorm(cfg.hidden_size, cfg.rms_norm_eps), attn,
                                   RMSNorm(cfg.hidden_size, cfg.rms_norm_eps), mlp))
    head = LMHead(cfg.vocab_size, cfg.hidden_size, tied_to=embed if cfg.tie_word_embeddings else None)
    return DecoderModel(cfg, embed, rotary, layers, RMSNorm(cfg.hidden_size, cfg.rms_norm_eps), head,
                        max_positions=cfg.max_position_embeddings)


register_architecture("Qwen3ForCausalLM", Qwen3Config, build_qwen3)
