"""The dense Llama-3 decoder (``LlamaForCausalLM``) put together from the parts.

Layer layout and checkpoint names follow
crates/infer-worker/src/models/decoder.rs:214-410 and
crates/infer-worker/src/models/llama3.rs:12-24.
"""
from __future__ import annotations

from ..config.model_config import LlamaConfig
from ..config.registry import register_architecture
from ..parts import (Embedding, LMHead, PagedAttention, PreNormBlock, RMSNorm,
                     RotaryEmbedding, SwiGLUMLP)
from .decoder import DecoderModel


def build_llama(cfg: LlamaConfig) -> DecoderModel:
    rope = RotaryEmbedding(cfg.head_dim, cfg.rope_theta, cfg.rope_scaling)
    embed = Embedding(cfg.vocab_size, cfg.hidden_size)
    layers = []
    for _ in range(cfg.num_hidden_layers):
        layers.append(PreNormBlock(
            cfg.hidden_size,
            RMSNorm(cfg.hidden_size, cfg.rms_norm_eps),
            PagedAttention(cfg.hidden_size, cfg.num_attention_heads, cfg.num_key_value_heads,
                           cfg.head_dim, pos_enc=rope),
            RMSNorm(cfg.hidden_size, cfg.rms_norm_eps),
            SwiGLUMLP(cfg.hidden_size, cfg.intermediate_size)))
    head = LMHead(cfg.vocab_size, cfg.hidden_size,
                  tied_to=embed if cfg.tie_word_embeddings else None)
    return DecoderModel(cfg, embed, layers, RMSNorm(cfg.hidden_size, cfg.rms_norm_eps), head,
                        position_encodings=[rope])


register_architecture("LlamaForCausalLM", LlamaConfig, build_llama, model_type="llama")
