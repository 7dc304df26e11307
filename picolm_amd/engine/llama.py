"""The dense Llama decoder as a list of parts (picolm/model_core.c runs this architecture:
RMSNorm, rotary GQA attention, SwiGLU, pre-norm residual blocks, optional tied head), and
its entry in the architecture registry."""
from __future__ import annotations

from ..config import LlamaConfig, register_architecture
from ..parts import (Attention, LMHead, PreNormBlock, RMSNorm, RotaryEmbedding, SwiGLU, TokenEmbedding)
from .model import DecoderModel


def build_llama(cfg: LlamaConfig) -> DecoderModel:
    D = cfg.hidden_size
    rotary = RotaryEmbedding(cfg.head_dim, cfg.rope_theta, cfg.rope_scaling, cfg.rope_style)
    blocks = []
    for l in range(cfg.num_hidden_layers):
        p = f"model.layers.{l}."
        blocks.append(PreNormBlock(
            RMSNorm(p + "input_layernorm.weight", D, cfg.rms_norm_eps),
            Attention(p + "self_attn.", D, cfg.num_attention_heads, cfg.num_key_value_heads, cfg.head_dim,
                      position=rotary),
            RMSNorm(p + "post_attention_layernorm.weight", D, cfg.rms_norm_eps),
            SwiGLU(p + "mlp.", D, cfg.intermediate_size)))
    emb = TokenEmbedding("model.embed_tokens.weight", cfg.vocab_size, D)
    return DecoderModel(cfg, emb, blocks, RMSNorm("model.norm.weight", D, cfg.rms_norm_eps),
                        LMHead("lm_head.weight", cfg.vocab_size, D, emb, cfg.tie_word_embeddings))


register_architecture("LlamaForCausalLM", LlamaConfig.from_dict, build_llama, replace=True)
