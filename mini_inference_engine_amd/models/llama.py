"""Llama dense decoder assembled from parts.

Layer formulas and tensor names as inference_engine/model.py:96-113,161-185:
per layer input_layernorm -> self_attn (q/k/v/o_proj, rotary half-split, GQA,
scale 1/sqrt(head_dim)) -> post_attention_layernorm -> mlp (gate/up/down_proj,
SiLU); model.norm; lm_head or the tied embedding.  Everything here is
construction: sizes and constants come from LlamaConfig only.
"""
from __future__ import annotations

from ..config.model_config import LlamaConfig
from ..config.registry import register_architecture
from ..parts import (Attention, DecoderSpec, Embedding, LMHead, PreNormBlock, RMSNorm, RotaryHalfSplit, SwiGLU)


def build_llama(cfg: LlamaConfig) -> DecoderSpec:
    h = cfg.hidden_size
    rope = RotaryHalfSplit(cfg.head_dim, cfg.rope_theta, cfg.max_position_embeddings)
    layers = []
    for i in range(cfg.num_hidden_layers):
        p = f"model.layers.{i}"
        layers.append(PreNormBlock(
            norm_mixer=RMSNorm(h, cfg.rms_norm_eps, f"{p}.input_layernorm.weight"),
            mixer=Attention(h, cfg.num_attention_heads, cfg.num_key_value_heads, cfg.head_dim,
                            scale=cfg.head_dim ** -0.5, position=rope, prefix=f"{p}.self_attn"),
            norm_feed_forward=RMSNorm(h, cfg.rms_norm_eps, f"{p}.post_attention_layernorm.weight"),
            feed_forward=SwiGLU(h, cfg.intermediate_size, prefix=f"{p}.mlp"),
        ))
    embedding = Embedding(cfg.vocab_size, h, "model.embed_tokens.weight")
    head = LMHead(cfg.vocab_size, h, "lm_head.weight", tied_to=embedding if cfg.tie_word_embeddings else None)
    ignore = [r".*\.rotary_emb\.inv_freq"]
    if cfg.tie_word_embeddings:
        ignore.append(r"lm_head\.weight")
    return DecoderSpec(embedding=embedding, layers=layers, final_norm=RMSNorm(h, cfg.rms_norm_eps, "model.norm.weight"),
                       head=head, ignore_tensors=tuple(ignore), eos_token_id=cfg.eos_token_id,
                       max_position=cfg.max_position_embeddings, vocab_size=cfg.vocab_size)


register_architecture("LlamaForCausalLM", LlamaConfig, build_llama, model_type="llama", replace=True)
